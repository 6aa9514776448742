"""GPU parity of the gemma3-style variant of the decode path (torch/io/gguf_model.h:74-88, :184-197): embedding rows
times sqrt(hidden), tanh-GELU gate, RMSNorm of each branch's output before the residual add, and alternating layers --
local ones attend to the last swa_window positions and rotate with their own base, global ones see everything and
rotate with linearly scaled positions.  The compiled reference's forward_decode_cpu run of synth.tiny_gemma is
golden_gemma.npz.  Bars are those of the qwen3-style tests."""
import os

import numpy as np
import pytest
import torch

from conftest import bits
from prometorch_amd import gguf, ops
from prometorch_amd.testing import gguf_writer, synth
from test_gpu_decode import check_step_errors
from test_gpu_llama import follow_sensitive
from test_gpu_prefill import check_kv_rows, check_logits

pytestmark = pytest.mark.gpu


def cu(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


@pytest.fixture(scope="module")
def golden_gemma():
    return np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "golden_gemma.npz"))


def tiny_gemma_with_cache(seeds, n=19):
    cfg, layers, head = synth.tiny_gemma(seeds["tiny"])
    kv = [synth.make_kv_prefill(seeds["tiny"], i, cfg, n) for i in range(cfg["n_layers"])]
    return cfg, layers, head, kv


def test_gelu_mul_rms_norm_add_and_scale(dev, po):
    r = synth.rng_for(93)
    gate = (3 * r.standard_normal(9728, dtype=np.float32)).astype(np.float32)
    up = r.standard_normal(9728, dtype=np.float32)
    want = gate.copy()
    po.lib().po_gelu_mul.argtypes = [po._vp, po._vp, po._i64]
    po.lib().po_gelu_mul(po._p(want), po._p(up), want.size)
    out = torch.empty(9728, device="cuda")
    ops.gelu_mul(cu(gate), cu(up), out, 9728)
    assert np.abs(out.cpu().numpy() - want).max() <= 2e-6 * np.abs(want).max()   # tanhf of the device library
    for rows, H in ((1, 2560), (5, 256)):
        h = r.standard_normal((rows, H), dtype=np.float32)
        x = r.standard_normal((rows, H), dtype=np.float32)
        w = (1 + 0.1 * r.standard_normal(H, dtype=np.float32)).astype(np.float32)
        dx = cu(x)
        ops.rms_norm_add(cu(h), cu(w), dx, rows, H, 1e-6)
        want = np.stack([x[i] + po.rmsnorm(h[i], w, 1e-6, seq=False) for i in range(rows)])
        assert np.abs(dx.cpu().numpy() - want).max() <= 2e-6 * np.abs(want).max()
    v = r.standard_normal(2560, dtype=np.float32)
    dv = cu(v)
    ops.scale(dv, float(np.sqrt(np.float32(2560))), 2560)
    assert np.array_equal(bits(dv.cpu().numpy()), bits(v * np.sqrt(np.float32(2560))))


@pytest.mark.parametrize("kv_fp16", [True, False])
@pytest.mark.parametrize("nh,nkv,hd,past,window", [(32, 8, 128, 2048, 1024), (4, 2, 64, 19, 8), (8, 4, 128, 130, 64),
                                                  (8, 8, 128, 5, 8), (16, 2, 64, 200, 1), (32, 8, 128, 511, 512),
                                                  (8, 4, 256, 2048, 1024), (2, 1, 256, 19, 8), (8, 4, 256, 30, 0), (6, 2, 256, 62, 0),
                                                  # heads of 256 with 1 and 4 query heads per kv head (matrix-core kernel, chunk
                                                  # edge crossed), with 5 (the vector kernel) and beyond 4096 positions (the same)
                                                  (4, 4, 256, 127, 0), (4, 1, 256, 63, 40), (5, 1, 256, 70, 0), (2, 1, 256, 5000, 300), (4, 1, 256, 8190, 0),
                                                  # caches beyond 4096 positions: the looping kernel (several chunks per workgroup,
                                                  # some or all of them in front of the window)
                                                  (8, 2, 128, 9000, 1024), (4, 2, 64, 5000, 100), (8, 4, 128, 8200, 7000)])
def test_attn_decode_fused_window_vs_oracle(dev, po, kv_fp16, nh, nkv, hd, past, window):
    """QK-norm + NeoX rotation + KV append + attention over the last `window` positions + merge, three tokens in a row:
    chunks wholly in front of the window are skipped, the chunk the window starts in is masked position by position."""
    max_seq = ((past + 3 + 63) // 64 + 1) * 64
    r = synth.rng_for(48, nh, hd, past)
    kvd = nkv * hd
    kf = r.standard_normal((max_seq, kvd), dtype=np.float32).astype(np.float16).astype(np.float32)
    vf = r.standard_normal((max_seq, kvd), dtype=np.float32).astype(np.float16).astype(np.float32)
    dt = torch.float16 if kv_fp16 else torch.float32
    Kc, Vc = cu(kf).to(dt), cu(vf).to(dt)
    Kc[past:] = float("nan")
    Vc[past:] = float("nan")
    S = ops.flash_decode_num_splits(max_seq)
    pO = torch.full((S * nh * hd,), float("nan"), device="cuda")
    pL = torch.full((S * nh,), float("nan"), device="cuda")
    pM = torch.full((S * nh,), float("nan"), device="cuda")
    table = ops.rope_table(max_seq, hd, 1e4).cuda()
    O = torch.empty(nh * hd, device="cuda")
    d_past = torch.zeros(1, dtype=torch.int64, device="cuda")
    scale = 1.0 / np.sqrt(hd)
    qw = (1 + 0.1 * r.standard_normal(hd, dtype=np.float32)).astype(np.float32)
    kw = (1 + 0.1 * r.standard_normal(hd, dtype=np.float32)).astype(np.float32)
    for step in range(3):
        pos = past + step
        q = synth.make_x(r, nh * hd).astype(np.float32)
        k = synth.make_x(r, kvd).astype(np.float32)
        v = synth.make_x(r, kvd)
        qn = np.concatenate([po.rmsnorm(q[h * hd:(h + 1) * hd], qw, 1e-6, seq=False) for h in range(nh)])
        kn = np.concatenate([po.rmsnorm(k[h * hd:(h + 1) * hd], kw, 1e-6, seq=False) for h in range(nkv)])
        c, s = po.rope_tables(pos, hd, 1e4)
        qr, kr = po.rope_neox(qn, kn, c, s, nh, nkv, hd)
        kf[pos] = kr.astype(np.float16).astype(np.float32) if kv_fp16 else kr
        vf[pos] = v.astype(np.float16).astype(np.float32) if kv_fp16 else v
        t_start = max(0, pos + 1 - window) if window else 0
        want = np.concatenate([po.attn_head(qr[h * hd:(h + 1) * hd], kf, vf, pos + 1, kvd, hd, scale,
                                            col0=(h // (nh // nkv)) * hd, t_start=t_start) for h in range(nh)])
        full = np.concatenate([po.attn_head(qr[h * hd:(h + 1) * hd], kf, vf, pos + 1, kvd, hd, scale,
                                            col0=(h // (nh // nkv)) * hd) for h in range(nh)])
        d_past.fill_(pos)
        ops.attn_decode_fused(cu(q), cu(k), cu(v), cu(qw), cu(kw), Kc, Vc, O, pO, pL, pM, table, nh, nkv, hd, d_past,
                              max_seq, scale, 1e-6, kv_fp16=kv_fp16, window=window)
        torch.cuda.synchronize()
        got = O.cpu().numpy()
        assert np.all(np.isfinite(got)), (step, pos)
        assert np.abs(got - want).max() <= 3e-5 * max(np.abs(want).max(), 1e-3) + 1e-6, (step, pos)
        if t_start > 0 and window > 0:
            assert np.abs(got - full).max() > 1e-3 * np.abs(full).max()   # the window does cut something off
        kf[pos] = Kc[pos].float().cpu().numpy()


@pytest.mark.parametrize("kv_fp16", [True, False])
@pytest.mark.parametrize("rows,nh,nkv,hd,pos0,window", [(23, 4, 2, 64, 0, 8), (40, 8, 4, 128, 100, 64), (7, 8, 8, 128, 30, 1),
                                                       (64, 16, 4, 64, 0, 1024),
                                                       # the matrix-core kernel with a window: its lower edge inside the walk (both
                                                       # wave-group counts), windows narrower than a tile and than a row block,
                                                       # 3 / 7 query heads per kv head
                                                       (300, 8, 4, 128, 700, 256), (200, 32, 8, 128, 2000, 1024), (130, 6, 2, 64, 50, 40),
                                                       (96, 4, 4, 128, 0, 33), (150, 14, 2, 64, 400, 5), (64, 8, 8, 64, 1000, 512),
                                                       (20, 8, 4, 256, 100, 64), (140, 8, 4, 256, 900, 300), (70, 4, 4, 256, 0, 20),
                                                       (256, 8, 4, 256, 1500, 1024)])
def test_prefill_attention_window_vs_oracle(dev, po, kv_fp16, rows, nh, nkv, hd, pos0, window):
    """fp16 cache and 16 or more rows: the matrix-core kernel (bar 1e-3 of the output's maximum, as without a window);
    otherwise the fp32 kernel (3e-5)."""
    r = synth.rng_for(49, rows, hd, pos0)
    kvd, max_seq = nkv * hd, pos0 + rows + 3
    kf = r.standard_normal((max_seq, kvd), dtype=np.float32).astype(np.float16).astype(np.float32)
    vf = r.standard_normal((max_seq, kvd), dtype=np.float32).astype(np.float16).astype(np.float32)
    q = r.standard_normal((rows, nh * hd), dtype=np.float32)
    dt = torch.float16 if kv_fp16 else torch.float32
    O = torch.empty(rows, nh * hd, device="cuda")
    scale = 1.0 / np.sqrt(hd)
    ops.prefill_attention_window(cu(q), cu(kf).to(dt), cu(vf).to(dt), O, rows, nh, nkv, hd, pos0, max_seq, scale, kv_fp16, window)
    got = O.cpu().numpy()
    for m in range(rows):
        T = pos0 + m + 1
        want = np.concatenate([po.attn_head(q[m, h * hd:(h + 1) * hd], kf, vf, T, kvd, hd, scale, col0=(h // (nh // nkv)) * hd,
                                            t_start=max(0, T - window)) for h in range(nh)])
        tol = 1e-3 if (kv_fp16 and rows >= 16) else 3e-5
        assert np.abs(got[m] - want).max() <= tol * max(np.abs(want).max(), 1e-3) + 1e-6, m


@pytest.mark.parametrize("use_graph", [False, True])
def test_gemma_teacher_forced_vs_reference_golden(dev, golden_gemma, seeds, use_graph):
    """16 distinct seeded ids fed step by step (the greedy run of this model repeats one id): argmax and logits of every step
    against the compiled reference's run of the same feed."""
    from prometorch_amd.decode import Decoder
    cfg, layers, head, kv = tiny_gemma_with_cache(seeds)
    dec = Decoder(cfg, layers, head, max_seq=64, kv_fp16=False, use_graph=use_graph)
    for i, (k, v) in enumerate(kv):
        dec.set_kv(i, k, v)
    dec.set_past_len(19)
    errs = []
    for st, t in enumerate(int(t) for t in golden_gemma["forced_feed"]):
        tok = dec.step(t)
        ref = golden_gemma["forced_logits"][st]
        errs.append(np.abs(dec.logits() - ref).max() / ref.std())
        srt = np.sort(ref)
        if (srt[-1] - srt[-2]) / ref.std() > 2 * max(errs[-1], 1e-4):
            assert tok == int(golden_gemma["forced_tokens"][st]), (st, errs[-1])
    check_step_errors(errs)
    dec.close()


@pytest.mark.parametrize("use_graph", [False, True])
def test_gemma_decode_fp32_kv_vs_reference_golden(dev, golden_gemma, seeds, use_graph):
    from prometorch_amd.decode import Decoder
    cfg, layers, head, kv = tiny_gemma_with_cache(seeds)
    dec = Decoder(cfg, layers, head, max_seq=64, kv_fp16=False, use_graph=use_graph)
    for i, (k, v) in enumerate(kv):
        dec.set_kv(i, k, v)
    dec.set_past_len(19)
    tok, errs = 3, []
    for st in range(16):
        tok = dec.step(tok)
        ref = golden_gemma["logits"][st]
        errs.append(np.abs(dec.logits() - ref).max() / ref.std())
        assert tok == int(golden_gemma["tokens"][st]), st
    check_step_errors(errs)
    dec.close()


@pytest.mark.parametrize("past", [19, 3])
def test_gemma_decode_fp16_kv_vs_oracle_and_chained_greedy(dev, po, seeds, past):
    """past = 3: the window of 8 is crossed during the run."""
    from prometorch_amd.decode import Decoder
    cfg, layers, head, kv = tiny_gemma_with_cache(seeds, past)
    om = po.OracleModel(cfg, layers, head, 64, kv_fp16=True)
    dec = Decoder(cfg, layers, head, max_seq=64, kv_fp16=True, use_graph=True)
    dec2 = Decoder(cfg, layers, head, max_seq=64, kv_fp16=True, use_graph=True)
    for i, (k, v) in enumerate(kv):
        om.set_kv(i, k, v)
        dec.set_kv(i, k, v)
        dec2.set_kv(i, k, v)
    dec.set_past_len(past)
    dec2.set_past_len(past)
    tok_o = tok_g = 3
    want, errs = [], []
    for st in range(24):
        tok_o = om.step(tok_o)
        tok_g = dec.step(tok_g)
        want.append(tok_o)
        errs.append(np.abs(dec.logits() - om.logits).max() / om.logits.std())
        assert tok_g == tok_o, st
    check_step_errors(errs)
    assert dec2.greedy(3, 24) == want
    dec.close()
    dec2.close()


@pytest.mark.parametrize("shape", ["tiny", "4b_layers", "hidden_4096", "hidden_4352"])
def test_step_that_defers_the_post_ffn_norm_matches_the_traced_step(dev, seeds, shape):
    """A plain step leaves the post-norm and residual add of a layer's feed-forward branch to the prologue of the next layer's
    q / k / v launch; a traced step runs each as a launch of its own.  Same state, same token: the logits agree to the
    bars of a decode step (the two sums of squares are taken in different orders, nothing else differs), and the traced
    residual stream after the last layer is what the plain step's final norm saw (hidden = RMSNorm of it)."""
    from prometorch_amd.decode import Decoder
    if shape == "tiny":
        cfg, layers, head = synth.tiny_gemma(seeds["tiny"])
        past, max_seq = 19, 64
    elif shape.startswith("hidden_"):
        # 4096 values: the longest vector the q / k / v prologue applies the post-norm to; 4352: one block beyond, every
        # post-norm a launch of its own (the two step forms then run the same launches)
        cfg = dict(synth.TINY, hidden=int(shape[7:]), n_layers=3, scale_embeddings=True, ffn_gelu=True, swa_window=8,
                   swa_pattern=3, rope_swa_base=1.0e4, rope_scale=8.0)
        layers = [synth.make_layer(seeds["tiny"], i, cfg) for i in range(cfg["n_layers"])]
        for i, L in enumerate(layers):
            g = synth.rng_for(seeds["tiny"], 6, i)
            for name in ("post_attn_norm", "post_ffn_norm"):
                L[name] = (np.float32(0.5) * (np.float32(1.0) + np.float32(0.1) * g.standard_normal(cfg["hidden"], dtype=np.float32))).astype(np.float32)
        head = synth.make_head(seeds["tiny"], cfg)
        past, max_seq = 19, 64
    else:
        cfg, layers, head = synth.gemma3_4b_like(seeds["cfg4"], n_layers=3, vocab=4096)
        past, max_seq = 300, 512
    decs = [Decoder(cfg, layers, head, max_seq=max_seq, kv_fp16=True, use_graph=g) for g in (False, True, False)]
    for d in decs:
        for i in range(cfg["n_layers"]):
            d.set_kv(i, *synth.make_kv_prefill(seeds["tiny"], i, cfg, past))
        d.set_past_len(past)
    tok, errs = 5, []
    for st in range(6):
        t_eager, t_graph = decs[0].step(tok), decs[1].step(tok)
        t_trace, trace = decs[2].step_trace(tok)
        ref = decs[2].logits()
        spread = ref.std()
        assert np.array_equal(decs[0].logits(), decs[1].logits()), st      # eager and graph replay: the same launches
        err = np.abs(decs[0].logits() - ref).max() / spread
        errs.append(err)
        x = trace[-1, 1].astype(np.float64)
        want_hidden = x / np.sqrt((x * x).mean() + cfg["eps"]) * head["out_norm"].astype(np.float64)
        assert np.abs(decs[0].hidden() - want_hidden).max() <= 2e-2 * np.abs(want_hidden).max(), st
        srt = np.sort(ref)
        if (srt[-1] - srt[-2]) / spread > 2 * max(err, 1e-4):
            assert t_eager == t_trace == t_graph, st
        tok = t_trace
    check_step_errors(errs)
    for d in decs:
        d.close()


@pytest.mark.parametrize("feature", ["scale_embeddings", "ffn_gelu", "swa_window", "rope_swa_base", "post_attn_norm", "post_ffn_norm"])
def test_gemma_features_are_not_ignored(dev, seeds, golden_gemma, feature):
    from prometorch_amd.decode import Decoder
    cfg, layers, head, kv = tiny_gemma_with_cache(seeds)
    if feature.startswith("post_"):
        layers = [{k: v for k, v in L.items() if k != feature} for L in layers]
    else:
        cfg = dict(cfg, **{feature: {"scale_embeddings": False, "ffn_gelu": False, "swa_window": 0, "rope_swa_base": 1.0e6}[feature]})
    dec = Decoder(cfg, layers, head, max_seq=64, kv_fp16=False, use_graph=False)
    for i, (k, v) in enumerate(kv):
        dec.set_kv(i, k, v)
    dec.set_past_len(19)
    dec.step(3)
    ref = golden_gemma["logits"][0]
    assert np.abs(dec.logits() - ref).max() > 1e-2 * ref.std()
    dec.close()


@pytest.mark.parametrize("kv_fp16", [True, False])
@pytest.mark.parametrize("pos0,n,chunk", [(0, 23, 0), (0, 23, 7), (19, 12, 5)])
def test_gemma_prefill_vs_oracle_token_by_token(dev, po, seeds, kv_fp16, pos0, n, chunk):
    from prometorch_amd.decode import Decoder
    cfg, layers, head = synth.tiny_gemma(seeds["tiny"])
    om = po.OracleModel(cfg, layers, head, 64, kv_fp16=kv_fp16)
    dec = Decoder(cfg, layers, head, max_seq=64, kv_fp16=kv_fp16, use_graph=True)
    if pos0:
        for i in range(cfg["n_layers"]):
            k, v = synth.make_kv_prefill(seeds["tiny"], i, cfg, pos0)
            om.set_kv(i, k, v)
            dec.set_kv(i, k, v)
        dec.set_past_len(pos0)
    prompt = [int(t) for t in synth.rng_for(69, pos0, n).integers(0, cfg["vocab"], n)]
    for t in prompt:
        tok_o = om.step(t)
    tok_g = dec.prefill(prompt, chunk_rows=chunk)
    for li in range(cfg["n_layers"]):
        for nm, gpu_c, cpu_c in (("k", dec.k_cache[li], om.k_cache[li]), ("v", dec.v_cache[li], om.v_cache[li])):
            check_kv_rows(gpu_c[pos0:pos0 + n].float().cpu().numpy(), cpu_c[pos0:pos0 + n], li, nm)
    check_logits(dec.logits(), om.logits, tok_g, tok_o, "prefill")
    follow_sensitive(dec, om, tok_o, 6)
    dec.close()


@pytest.mark.parametrize("kv_fp16", [True, False])
@pytest.mark.parametrize("nh,nkv,hd,past,window", [(8, 4, 256, 2048, 1024), (8, 4, 256, 2048, 0), (2, 1, 256, 19, 8), (4, 4, 128, 300, 100)])
def test_flash_decode_window_vs_oracle(dev, po, kv_fp16, nh, nkv, hd, past, window):
    """The plain split-KV attention (the path of 256-wide heads) over a window, with the Q8 copy of its output."""
    T = past + 1
    max_seq = ((T + 127) // 64) * 64
    r = synth.rng_for(50, nh, hd, past)
    kvd = nkv * hd
    kf = r.standard_normal((max_seq, kvd), dtype=np.float32).astype(np.float16).astype(np.float32)
    vf = r.standard_normal((max_seq, kvd), dtype=np.float32).astype(np.float16).astype(np.float32)
    q = synth.make_x(r, nh * hd)
    scale = 1.0 / np.sqrt(hd)
    t_start = max(0, T - window) if window else 0
    want = np.concatenate([po.attn_head(q[h * hd:(h + 1) * hd], kf, vf, T, kvd, hd, scale, col0=(h // (nh // nkv)) * hd,
                                        t_start=t_start) for h in range(nh)])
    dt = torch.float16 if kv_fp16 else torch.float32
    Kc, Vc = cu(kf).to(dt), cu(vf).to(dt)
    Kc[T:] = float("nan")
    Vc[T:] = float("nan")
    S = ops.flash_decode_num_splits(max_seq)
    pO = torch.full((S * nh * hd,), float("nan"), device="cuda")
    pL = torch.full((S * nh,), float("nan"), device="cuda")
    pM = torch.full((S * nh,), float("nan"), device="cuda")
    O = torch.empty(nh * hd, device="cuda")
    q8 = torch.zeros(ops.q8_bytes(nh * hd), dtype=torch.uint8, device="cuda")
    d_past = torch.tensor([past], dtype=torch.int64, device="cuda")
    ops.flash_decode_window(cu(q), Kc, Vc, O, pO, pL, pM, nh, nkv, hd, d_past, max_seq, scale, kv_fp16=kv_fp16, window=window, o_q8=q8)
    torch.cuda.synchronize()
    got = O.cpu().numpy()
    assert np.all(np.isfinite(got))
    assert np.abs(got - want).max() <= 3e-5 * max(np.abs(want).max(), 1e-3) + 1e-6
    K = nh * hd
    raw = q8.cpu().numpy()
    qs = raw[:K].view(np.int8).astype(np.float32)
    d = raw[K:K + 4 * (K // 32)].view(np.float32)
    assert np.abs(qs * np.repeat(d, 32) - got).max() <= 0.51 * d.max()   # the Q8 blocks are this vector, rounded


@pytest.mark.parametrize("kv_fp16", [True, False])
def test_gemma_wide_heads_decode_and_prefill_vs_oracle(dev, po, seeds, kv_fp16):
    """head_dim 256 (gemma3's width): decode from a cache, chained greedy, and a prompt through the row-batched path."""
    from prometorch_amd.decode import Decoder
    cfg, layers, head = synth.tiny_gemma(seeds["tiny"], head_dim=256)
    kv = [synth.make_kv_prefill(seeds["tiny"], i, cfg, 19) for i in range(cfg["n_layers"])]
    om = po.OracleModel(cfg, layers, head, 64, kv_fp16=kv_fp16)
    dec = Decoder(cfg, layers, head, max_seq=64, kv_fp16=kv_fp16, use_graph=True)
    dec2 = Decoder(cfg, layers, head, max_seq=64, kv_fp16=kv_fp16, use_graph=True)
    for i, (k, v) in enumerate(kv):
        om.set_kv(i, k, v)
        dec.set_kv(i, k, v)
        dec2.set_kv(i, k, v)
    dec.set_past_len(19)
    dec2.set_past_len(19)
    tok_o = tok_g = 3
    want, errs = [], []
    for st in range(16):
        tok_o = om.step(tok_o)
        tok_g = dec.step(tok_g)
        want.append(tok_o)
        errs.append(np.abs(dec.logits() - om.logits).max() / om.logits.std())
        assert tok_g == tok_o, st
    check_step_errors(errs)
    assert dec2.greedy(3, 16) == want
    dec.close()
    dec2.close()
    om = po.OracleModel(cfg, layers, head, 64, kv_fp16=kv_fp16)
    dec = Decoder(cfg, layers, head, max_seq=64, kv_fp16=kv_fp16, use_graph=True)
    prompt = [int(t) for t in synth.rng_for(70).integers(0, cfg["vocab"], 23)]
    for t in prompt:
        tok_o = om.step(t)
    tok_g = dec.prefill(prompt, chunk_rows=7)
    for li in range(cfg["n_layers"]):
        for nm, gpu_c, cpu_c in (("k", dec.k_cache[li], om.k_cache[li]), ("v", dec.v_cache[li], om.v_cache[li])):
            check_kv_rows(gpu_c[:23].float().cpu().numpy(), cpu_c[:23], li, nm)
    check_logits(dec.logits(), om.logits, tok_g, tok_o, "prefill")
    follow_sensitive(dec, om, tok_o, 6)
    dec.close()


def test_gemma3_gguf_file_decodes_like_direct_decoder(dev, seeds, golden_gemma, tmp_path):
    """general.architecture = gemma3: sliding_window / sliding_window_pattern / rope.freq_base_swa / rope.scaling.* keys and
    the post_attention_norm / post_ffw_norm vectors are read; scaled embeddings and the GELU gate follow from the name."""
    from prometorch_amd.decode import Decoder
    cfg, layers, head, kv = tiny_gemma_with_cache(seeds)
    path = str(tmp_path / "tiny_gemma3.gguf")
    gguf_writer.model_to_gguf(path, cfg, layers, head, arch="gemma3")
    m = gguf.GGUFModel(path, max_seq=64, kv_fp16=False)
    for key in ("scale_embeddings", "ffn_gelu", "swa_window", "swa_pattern", "rope_swa_base", "rope_scale"):
        assert m.cfg[key] == cfg[key], key
    assert m.layer(2).post_attn_norm and m.layer(2).post_ffn_norm and m.layer(2).q_norm
    d = Decoder(cfg, layers, head, max_seq=64, kv_fp16=False)
    for i, (k, v) in enumerate(kv):
        m.set_kv(i, k, v)
        d.set_kv(i, k, v)
    m.set_past_len(19)
    d.set_past_len(19)
    tm = td = 3
    for st in range(16):
        tm = m.step(tm)
        td = d.step(td)
        assert tm == td == int(golden_gemma["tokens"][st]), st
        assert np.array_equal(bits(m.logits()), bits(d.logits())), st
    m.close()
    d.close()
    # without the pattern key every sixth layer is global: the four-layer model is all local then
    p2 = str(tmp_path / "default_pattern.gguf")
    gguf_writer.model_to_gguf(p2, dict(cfg, swa_pattern=6), layers, head, arch="gemma3")
    m2 = gguf.GGUFModel(p2, max_seq=64, kv_fp16=False)
    assert m2.cfg["swa_pattern"] == 6
    m2.close()


def test_gemma3_4b_layer_shapes_decode_and_prefill_vs_oracle(dev, po, seeds):
    """Two layers of Gemma-3-4B size (2560 hidden, 8 heads of 256 on 4 kv heads, 10240 intermediate, window 1024, bases
    1e4 / 1e6 with positions divided by 8) over a 32000-token vocabulary, the second layer global: 8 decode steps behind
    1100 cached positions (past the window) and a 40-token prompt, against the oracle."""
    from prometorch_amd.decode import Decoder
    from test_gpu_decode import LOGIT_TOL, LOGIT_TOL_FLIP
    from test_gpu_prefill import logit_errors
    cfg, layers, head = synth.gemma3_4b_like(seeds["cfg4"])
    cfg["swa_pattern"] = 2
    om = po.OracleModel(cfg, layers, head, 1280, kv_fp16=True)
    dec = Decoder(cfg, layers, head, max_seq=1280, kv_fp16=True, use_graph=True)
    for i in range(cfg["n_layers"]):
        k, v = synth.make_kv_prefill(seeds["cfg4"], i, cfg, 1100)
        om.set_kv(i, k, v)
        dec.set_kv(i, k, v)
    dec.set_past_len(1100)
    tok, errs = 11, []
    for st in range(8):
        tok_o = om.step(tok)
        tok_g = dec.step(tok)
        err, rms, margin = logit_errors(dec.logits(), om.logits)
        errs.append(err)
        if margin > 2 * err:
            assert tok_g == tok_o, (st, margin, err)
        tok = tok_o
    errs = np.asarray(errs)
    print("decode steps: logit err/std", np.array2string(errs, precision=2), flush=True)
    assert errs.max() <= LOGIT_TOL_FLIP and np.median(errs) <= LOGIT_TOL, errs
    prompt = [int(t) for t in synth.rng_for(72).integers(0, cfg["vocab"], 40)]
    for t in prompt:
        tok_o = om.step(t)
    tok_g = dec.prefill(prompt)
    for li in range(2):
        check_kv_rows(dec.k_cache[li][1108:1148].float().cpu().numpy(), om.k_cache[li][1108:1148], li, "k")
        check_kv_rows(dec.v_cache[li][1108:1148].float().cpu().numpy(), om.v_cache[li][1108:1148], li, "v")
    check_logits(dec.logits(), om.logits, tok_g, tok_o, "prefill")
    dec.close()
