"""GPU parity of the qwen2-style variant of the decode path: bias vectors added to the q / k / v projections before
the rotation (torch/io/gguf_model.h:2768-2779 on the GPU, :3413-3438 on the CPU), no per-head QK-norm, NeoX rotation
pairs.  The compiled reference's forward_decode_cpu run of synth.tiny_qwen2 is golden_qwen2.npz.  Bars are those of
the qwen3-style tests: tokens identical, logits within LOGIT_TOL of the spread (decode), the prefill bars of
test_gpu_prefill for the prompt path, bit-identical results between a .gguf load and the direct decoder."""
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
def golden_qwen2():
    return np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "golden_qwen2.npz"))


def tiny_qwen2_with_cache(seeds, n=19):
    cfg, layers, head = synth.tiny_qwen2(seeds["tiny"])
    kv = [synth.make_kv_prefill(seeds["tiny"], i, cfg, n) for i in range(cfg["n_layers"])]
    return cfg, layers, head, kv


@pytest.mark.parametrize("rows,qd,kvd", [(1, 4096, 1024), (7, 256, 128), (33, 512, 512)])
def test_add_qkv_bias_is_one_fp32_add_per_element(dev, rows, qd, kvd):
    r = synth.rng_for(91, rows, qd)
    Q, K, V = (r.standard_normal((rows, n), dtype=np.float32) for n in (qd, kvd, kvd))
    bq, bk, bv = (r.standard_normal(n, dtype=np.float32) for n in (qd, kvd, kvd))
    dQ, dK, dV = cu(Q), cu(K), cu(V)
    ops.add_qkv_bias(dQ, dK, dV, cu(bq), cu(bk), cu(bv), rows, qd, kvd)
    for got, want in ((dQ, Q + bq), (dK, K + bk), (dV, V + bv)):
        assert np.array_equal(bits(got.cpu().numpy()), bits(want))


@pytest.mark.parametrize("nh,nkv,hd,past,max_seq,interleaved", [
    (28, 4, 128, 2100, 2304, 0), (12, 2, 128, 300, 512, 0), (14, 2, 64, 63, 128, 0), (4, 4, 64, 0, 64, 1),
    (28, 4, 128, 5000, 8192, 0), (16, 2, 64, 4097, 4224, 1)])
def test_attention_launch_that_adds_the_biases_equals_the_separate_add(dev, nh, nkv, hd, past, max_seq, interleaved):
    """With an fp16 cache and heads of 64 or 128 the decoder hands the bias vectors to the attention launch instead of
    running the bias kernel first (caches of up to 4096 positions and beyond: both kernels): output, its Q8 blocks and the
    appended cache rows are bit-identical to bias kernel + attention."""
    import ctypes as C
    from prometorch_amd import _lib
    L = _lib.load()
    vp = C.c_void_p
    tail = [C.c_int, C.c_int, C.c_int, vp, C.c_int, C.c_float, C.c_float, C.c_int, C.c_int, C.c_int]
    plain, fold = L.ptm_attn_decode_fused_q8, L.ptm_attn_decode_fused_bias
    plain.restype = fold.restype = C.c_int
    plain.argtypes = [vp] * 13 + tail + [vp]
    fold.argtypes = [vp] * 16 + tail + [C.c_int, vp]
    assert L.ptm_attn_decode_folds_bias(hd, 1) == 1 and L.ptm_attn_decode_folds_bias(256, 1) == 0
    assert L.ptm_attn_decode_folds_bias(hd, 0) == 0
    r = synth.rng_for(93, nh, hd, past)
    kvd, qd = nkv * hd, nh * hd
    K0 = r.standard_normal((max_seq, kvd), dtype=np.float32).astype(np.float16)
    V0 = r.standard_normal((max_seq, kvd), dtype=np.float32).astype(np.float16)
    S = ops.flash_decode_num_splits(max_seq)
    table = ops.rope_table(max_seq, hd, 1e6).cuda()
    d_past = torch.full((1,), past, dtype=torch.int64, device="cuda")
    Q, K, V = synth.make_x(r, qd) * 3, synth.make_x(r, kvd) * 3, synth.make_x(r, kvd)
    bq, bk, bv = synth.make_x(r, qd) * 2, synth.make_x(r, kvd) * 2, synth.make_x(r, kvd)
    p = lambda t: t.data_ptr()
    res = []
    for folded in (False, True):
        Kc, Vc = cu(K0), cu(V0)
        pO, pL, pM = torch.empty(S * qd, device="cuda"), torch.empty(S * nh, device="cuda"), torch.empty(S * nh, device="cuda")
        O = torch.empty(qd, device="cuda")
        q8 = torch.zeros(ops.q8_bytes(qd), dtype=torch.uint8, device="cuda")
        dQ, dK, dV, dbq, dbk, dbv = cu(Q), cu(K), cu(V), cu(bq), cu(bk), cu(bv)
        if folded:
            rc = fold(p(dQ), p(dK), p(dV), p(dbq), p(dbk), p(dbv), None, None, p(Kc), p(Vc), p(O), p(q8), p(pO), p(pL),
                      p(pM), p(table), nh, nkv, hd, p(d_past), max_seq, 1.0 / np.sqrt(hd), 1e-6, 0, 1, interleaved, 0, None)
        else:
            ops.add_qkv_bias(dQ, dK, dV, dbq, dbk, dbv, 1, qd, kvd)
            rc = plain(p(dQ), p(dK), p(dV), None, None, p(Kc), p(Vc), p(O), p(q8), p(pO), p(pL), p(pM), p(table), nh, nkv,
                       hd, p(d_past), max_seq, 1.0 / np.sqrt(hd), 1e-6, 0, 1, interleaved, None)
        assert rc == 0
        torch.cuda.synchronize()
        res.append((O.cpu().numpy(), q8.cpu().numpy(), Kc[past].cpu().numpy(), Vc[past].cpu().numpy()))
    assert np.isfinite(res[0][0]).all() and np.abs(res[0][0]).max() > 0
    for a, b in zip(*res):
        assert np.array_equal(a.view(np.uint8), b.view(np.uint8))
    # where the launch cannot add them it says so and launches nothing
    assert fold(16, 16, 16, 16, 16, 16, None, None, 16, 16, 16, None, 16, 16, 16, 16, 8, 4, 256, 16, 128, 1.0, 1e-6, 0, 1, 0, 0,
                None) == -4
    assert fold(16, 16, 16, 16, 16, 16, None, None, 16, 16, 16, None, 16, 16, 16, 16, 8, 4, 128, 16, 128, 1.0, 1e-6, 0, 0, 0, 0,
                None) == -4
    assert fold(16, 16, 16, 16, None, 16, None, None, 16, 16, 16, None, 16, 16, 16, 16, 8, 4, 128, 16, 128, 1.0, 1e-6, 0, 1, 0, 0,
                None) == -1


@pytest.mark.parametrize("use_graph", [False, True])
def test_qwen2_teacher_forced_vs_reference_golden(dev, golden_qwen2, seeds, use_graph):
    """16 distinct seeded ids fed step by step (the greedy run of this model repeats one id): argmax and logits of every step
    against the compiled reference's run of the same feed."""
    from prometorch_amd.decode import Decoder
    cfg, layers, head, kv = tiny_qwen2_with_cache(seeds)
    dec = Decoder(cfg, layers, head, max_seq=64, kv_fp16=False, use_graph=use_graph)
    for i, (k, v) in enumerate(kv):
        dec.set_kv(i, k, v)
    dec.set_past_len(19)
    errs = []
    for st, t in enumerate(int(t) for t in golden_qwen2["forced_feed"]):
        tok = dec.step(t)
        ref = golden_qwen2["forced_logits"][st]
        errs.append(np.abs(dec.logits() - ref).max() / ref.std())
        srt = np.sort(ref)
        if (srt[-1] - srt[-2]) / ref.std() > 2 * max(errs[-1], 1e-4):
            assert tok == int(golden_qwen2["forced_tokens"][st]), (st, errs[-1])
    check_step_errors(errs)
    dec.close()


@pytest.mark.parametrize("use_graph", [False, True])
def test_qwen2_decode_fp32_kv_vs_reference_golden(dev, golden_qwen2, seeds, use_graph):
    from prometorch_amd.decode import Decoder
    cfg, layers, head, kv = tiny_qwen2_with_cache(seeds)
    dec = Decoder(cfg, layers, head, max_seq=64, kv_fp16=False, use_graph=use_graph)
    for i, (k, v) in enumerate(kv):
        dec.set_kv(i, k, v)
    dec.set_past_len(19)
    tok, errs = 3, []
    for st in range(12):
        tok = dec.step(tok)
        ref = golden_qwen2["logits"][st]
        errs.append(np.abs(dec.logits() - ref).max() / ref.std())
        assert tok == int(golden_qwen2["tokens"][st]), st
    check_step_errors(errs)
    dec.close()


def test_qwen2_decode_fp16_kv_vs_oracle_and_chained_greedy(dev, po, seeds):
    from prometorch_amd.decode import Decoder
    cfg, layers, head, kv = tiny_qwen2_with_cache(seeds)
    om = po.OracleModel(cfg, layers, head, 64, kv_fp16=True)
    dec = Decoder(cfg, layers, head, max_seq=64, kv_fp16=True, use_graph=True)
    dec2 = Decoder(cfg, layers, head, max_seq=64, kv_fp16=True, use_graph=True)
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
    assert dec2.greedy(3, 24) == want
    # the appended K rows carry the k bias, the V rows the v bias
    for gpu_c, cpu_c in ((dec.k_cache[0], om.k_cache[0]), (dec.v_cache[1], om.v_cache[1])):
        got, ref = gpu_c[19:43].float().cpu().numpy(), cpu_c[19:43]
        assert np.abs(got - ref).max() <= 2e-3 * np.abs(ref).max()
    dec.close()
    dec2.close()


def test_qwen2_biases_are_not_ignored(dev, seeds, golden_qwen2):
    """The same weights without the bias vectors give other logits at the first step: the golden run exercises them."""
    from prometorch_amd.decode import Decoder
    cfg, layers, head, kv = tiny_qwen2_with_cache(seeds)
    bare = [{k: v for k, v in L.items() if not k.endswith("_bias")} for L in layers]
    dec = Decoder(cfg, bare, head, max_seq=64, kv_fp16=False, use_graph=False)
    for i, (k, v) in enumerate(kv):
        dec.set_kv(i, k, v)
    dec.set_past_len(19)
    dec.step(3)
    ref = golden_qwen2["logits"][0]
    assert np.abs(dec.logits() - ref).max() > 0.05 * ref.std()
    dec.close()


def test_decoder_wants_all_three_biases_or_none(dev, seeds):
    from prometorch_amd._lib import PtmError
    from prometorch_amd.decode import Decoder
    cfg, layers, head = synth.tiny_qwen2(seeds["tiny"])
    bad = [dict(L) for L in layers]
    bad[1]["v_bias"] = None
    with pytest.raises(PtmError) as e:
        Decoder(cfg, bad, head, max_seq=64, kv_fp16=False)
    assert e.value.code == -1


@pytest.mark.parametrize("kv_fp16", [True, False])
@pytest.mark.parametrize("pos0,n,chunk", [(0, 23, 0), (0, 23, 7), (19, 12, 5)])
def test_qwen2_prefill_vs_oracle_token_by_token(dev, po, seeds, kv_fp16, pos0, n, chunk):
    from prometorch_amd.decode import Decoder
    cfg, layers, head = synth.tiny_qwen2(seeds["tiny"])
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
    follow_sensitive(dec, om, tok_o, 6)
    dec.close()


def test_qwen2_gguf_file_decodes_like_direct_decoder(dev, seeds, golden_qwen2, tmp_path):
    """general.architecture = qwen2: blk.N.attn_{q,k,v}.bias vectors loaded, no QK-norm tensors, NeoX rotation."""
    from prometorch_amd.decode import Decoder
    cfg, layers, head, kv = tiny_qwen2_with_cache(seeds)
    path = str(tmp_path / "tiny_qwen2.gguf")
    gguf_writer.model_to_gguf(path, cfg, layers, head, arch="qwen2")
    f = gguf.GGUFFile(path)
    assert np.array_equal(f.tensor("blk.1.attn_k.bias")["data"].view(np.float32), layers[1]["k_bias"])
    f.close()
    m = gguf.GGUFModel(path, max_seq=64, kv_fp16=False)
    assert m.cfg["rope_interleaved"] is False
    assert m.layer(0).q_bias and m.layer(0).v_bias and not m.layer(0).q_norm
    d = Decoder(cfg, layers, head, max_seq=64, kv_fp16=False)
    for i, (k, v) in enumerate(kv):
        m.set_kv(i, k, v)
        d.set_kv(i, k, v)
    m.set_past_len(19)
    d.set_past_len(19)
    tm = td = 3
    for st in range(12):
        tm = m.step(tm)
        td = d.step(td)
        assert tm == td == int(golden_qwen2["tokens"][st]), st
        assert np.array_equal(bits(m.logits()), bits(d.logits())), st
    m.close()
    d.close()
    # a file with only two of the three bias vectors: missing tensor
    part = [dict(L) for L in layers]
    for L in part:
        L["v_bias"] = None
    p2 = str(tmp_path / "partial.gguf")
    gguf_writer.model_to_gguf(p2, cfg, part, head, arch="qwen2")
    from prometorch_amd._lib import PtmError
    with pytest.raises(PtmError) as e:
        gguf.GGUFModel(p2, max_seq=64)
    assert e.value.code == -10


def test_qwen25_7b_layer_shapes_decode_and_prefill_vs_oracle(dev, po, seeds):
    """Two layers of Qwen2.5-7B size (3584 hidden = 14 super-blocks, 18944 intermediate = 74, 28 query heads on 4 kv heads,
    biases) over a 32000-token vocabulary: 8 decode steps behind 300 cached positions and a 40-token prompt against the
    oracle.  Bars as for the Llama-3-8B-shaped test: the median step within LOGIT_TOL, every step within LOGIT_TOL_FLIP,
    tokens equal wherever the oracle's margin exceeds twice the error."""
    from prometorch_amd.decode import Decoder
    from test_gpu_decode import LOGIT_TOL, LOGIT_TOL_FLIP
    from test_gpu_prefill import logit_errors
    cfg, layers, head = synth.qwen25_7b_like(seeds["cfg4"])
    om = po.OracleModel(cfg, layers, head, 512, kv_fp16=True)
    dec = Decoder(cfg, layers, head, max_seq=512, kv_fp16=True, use_graph=True)
    for i in range(cfg["n_layers"]):
        k, v = synth.make_kv_prefill(seeds["cfg4"], i, cfg, 300)
        om.set_kv(i, k, v)
        dec.set_kv(i, k, v)
    dec.set_past_len(300)
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
    prompt = [int(t) for t in synth.rng_for(73).integers(0, cfg["vocab"], 40)]
    for t in prompt:
        tok_o = om.step(t)
    tok_g = dec.prefill(prompt)
    for li in range(2):
        check_kv_rows(dec.k_cache[li][308:348].float().cpu().numpy(), om.k_cache[li][308:348], li, "k")
        check_kv_rows(dec.v_cache[li][308:348].float().cpu().numpy(), om.v_cache[li][308:348], li, "v")
    err, rms, margin = logit_errors(dec.logits(), om.logits)
    print("prefill: logit err/std %.2e margin %.2e" % (err, margin), flush=True)
    dec.close()
