"""GPU parity of the prompt (prefill) path: the row-batched glue kernels against the oracle's pieces, and the whole
prefill against the oracle stepping the same prompt one token at a time -- which is what the reference's
forward(tokens, use_cache) computes row by row (torch/io/gguf_model.h:2510-2571; its M-row matmul is a loop of
GEMVs, :7029-7036).

Bars: embedding rows bit-exact; QK-norm/RoPE rows within 2e-6 of the row's maximum; attention within 1e-4; every
stage of a layer, fed the SAME input on both sides, within STAGE_TOL (GEMMs: fp16 rounding of both operands, 1e-2 is
the stated bar of the prefill GEMM; measured ~1e-3).

End to end the two paths cannot stay that close: each Q4_K matrix product rounds its activation vector to int8
(reference semantics), and a vector that differs by 1e-3 of a rounding step lands on the neighbouring level in
that fraction of its elements, each a full step (1/127 of the block maximum) apart.  Through a few such stages the
difference grows to the size of the Q8 rounding noise itself and stays there (it does not keep growing: measured
rms 3e-3..7e-3 of the logits' spread for 2 and for 36 layers).  test_q8_rounding_noise_floor_of_the_oracle shows
the same growth inside the CPU oracle alone when its input embedding is perturbed by the fp16 GEMM's error.  The
end-to-end bars are therefore on that scale: logits rms within E2E_RMS_TOL and max within E2E_MAX_TOL of the spread
of the oracle's logits, greedy tokens identical wherever the oracle's top-2 margin exceeds twice the logit error."""
import numpy as np
import pytest
import torch

from conftest import bits
from prometorch_amd import ops
from prometorch_amd.testing import synth
from prometorch_amd._lib import PtmError

pytestmark = pytest.mark.gpu

PREFILL_TOL = 1e-2   # a single GEMM, max |y - y_cpu| / rms(y_cpu)
STAGE_TOL = 5e-3     # one stage of a layer on identical inputs
E2E_RMS_TOL = 1e-2   # whole model: rms of the logit difference / std of the oracle's logits
E2E_MAX_TOL = 6e-2   # whole model: max of the same
# 1100+ rows: the worst of five prompt lengths (the median is held to E2E_RMS_TOL).  Measured: four lengths at 1.5e-3 .. 2.8e-3,
# the fifth (1100 tokens, a position where the int8 rounding noise tips a residual row) at 6.1e-2 .. 9.7e-2, against the oracle
# as against this decoder's own token-by-token run; the bar is that plus half again
LONG_RMS_WORST = 0.15


def cu(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


@pytest.mark.parametrize("tied_q6k", [True, False])
def test_embedding_rows_bit_exact(dev, po, tied_q6k):
    vocab, hidden, rows = 300, 512, 37
    r = synth.rng_for(61, tied_q6k)
    W = synth.make_weight(r, 14, vocab, hidden)
    table = po.dequant(14, W).reshape(vocab, hidden)
    toks = r.integers(0, vocab, rows).astype(np.int32)
    toks[0], toks[1] = 0, vocab - 1
    out = torch.full((rows, hidden), 7.0, device="cuda")
    if tied_q6k:
        ops.embedding_rows(None, cu(W), W.shape[1], cu(toks), rows, hidden, vocab, out)
    else:
        ops.embedding_rows(cu(table), None, 0, cu(toks), rows, hidden, vocab, out)
    torch.cuda.synchronize()
    assert np.array_equal(bits(out.cpu().numpy()), bits(table[toks]))


def test_embedding_rows_rejects_bad_arguments(dev):
    out = torch.zeros(4, 256, device="cuda")
    toks = torch.zeros(4, dtype=torch.int32, device="cuda")
    with pytest.raises(PtmError):
        ops.embedding_rows(None, None, 0, toks, 4, 256, 10, out)       # no table at all
    with pytest.raises(PtmError):
        ops.embedding_rows(None, out, 210, toks, 4, 200, 10, out)      # hidden not a multiple of 256 for Q6_K rows
    with pytest.raises(PtmError):
        ops.embedding_rows(out, None, 0, toks, 0, 256, 10, out)        # no rows


@pytest.mark.parametrize("kv_fp16", [True, False])
@pytest.mark.parametrize("nh,nkv,hd,pos0,rows", [(32, 8, 128, 2040, 9), (4, 2, 64, 0, 21), (8, 8, 128, 5, 3), (8, 4, 256, 5, 7),
                                                 (6, 2, 128, 3, 5),   # head counts that leave lanes of the last wave idle
                                                 (3, 1, 64, 0, 4),
                                                 (6, 2, 96, 3, 5)])   # a head width served by the one-wave-per-head kernel
def test_qknorm_rope_kvwrite_rows_vs_oracle(dev, po, kv_fp16, nh, nkv, hd, pos0, rows):
    max_seq = pos0 + rows + 3
    r = synth.rng_for(62, nh, hd, pos0)
    kvd = nkv * hd
    q = (r.standard_normal((rows, nh * hd), dtype=np.float32) * 4)
    k = (r.standard_normal((rows, kvd), dtype=np.float32) * 4)
    v = r.standard_normal((rows, kvd), dtype=np.float32)
    qw = (1 + 0.1 * synth.make_x(r, hd)).astype(np.float32)
    kw = (1 + 0.1 * synth.make_x(r, hd)).astype(np.float32)
    want_q, want_k = np.empty_like(q), np.empty_like(k)
    for m in range(rows):
        qn = np.concatenate([po.rmsnorm(q[m, h * hd:(h + 1) * hd], qw, 1e-6) for h in range(nh)])
        kn = np.concatenate([po.rmsnorm(k[m, h * hd:(h + 1) * hd], kw, 1e-6) for h in range(nkv)])
        c, s = po.rope_tables(pos0 + m, hd, 1e6)
        want_q[m], want_k[m] = po.rope_neox(qn, kn, c, s, nh, nkv, hd)
    dt = torch.float16 if kv_fp16 else torch.float32
    Kc = torch.zeros(max_seq, kvd, dtype=dt, device="cuda")
    Vc = torch.zeros(max_seq, kvd, dtype=dt, device="cuda")
    Q, K, V = cu(q), cu(k), cu(v)
    table = ops.rope_table(max_seq, hd, 1e6).cuda()
    ops.qknorm_rope_kvwrite_rows(Q, K, V, cu(qw), cu(kw), Kc, Vc, table, rows, nh, nkv, hd, pos0, max_seq, 1e-6, False,
                                 kv_fp16)
    torch.cuda.synchronize()
    assert np.abs(Q.cpu().numpy() - want_q).max() <= 2e-6 * np.abs(want_q).max()
    assert np.abs(K.cpu().numpy() - want_k).max() <= 2e-6 * np.abs(want_k).max()
    krows, vrows = Kc[pos0:pos0 + rows].float().cpu().numpy(), Vc[pos0:pos0 + rows].float().cpu().numpy()
    if kv_fp16:
        assert np.array_equal(vrows, v.astype(np.float16).astype(np.float32))
        assert np.array_equal(krows, K.cpu().numpy().astype(np.float16).astype(np.float32))
    else:
        assert np.array_equal(vrows, v) and np.array_equal(krows, K.cpu().numpy())
    # nothing outside the rows' own positions is written
    assert float(Kc[:pos0].abs().sum()) == 0 and float(Kc[pos0 + rows:].abs().sum()) == 0
    # rows that would land beyond the cache are an error, not a partial write
    with pytest.raises(PtmError):
        ops.qknorm_rope_kvwrite_rows(Q, K, V, cu(qw), cu(kw), Kc, Vc, table, rows, nh, nkv, hd, max_seq - rows + 1, max_seq,
                                     1e-6, False, kv_fp16)


def test_qknorm_rope_kvwrite_rows_without_norm_weights(dev, po):
    """Architectures without QK-norm (Llama): RoPE and the cache append only."""
    nh, nkv, hd, rows, pos0, max_seq = 8, 2, 128, 5, 11, 32
    r = synth.rng_for(63)
    q = r.standard_normal((rows, nh * hd), dtype=np.float32)
    k = r.standard_normal((rows, nkv * hd), dtype=np.float32)
    v = r.standard_normal((rows, nkv * hd), dtype=np.float32)
    want_q, want_k = np.empty_like(q), np.empty_like(k)
    for m in range(rows):
        c, s = po.rope_tables(pos0 + m, hd, 1e4)
        want_q[m], want_k[m] = po.rope_neox(q[m], k[m], c, s, nh, nkv, hd)
    Kc = torch.zeros(max_seq, nkv * hd, device="cuda")
    Vc = torch.zeros(max_seq, nkv * hd, device="cuda")
    Q, K = cu(q), cu(k)
    ops.qknorm_rope_kvwrite_rows(Q, K, cu(v), None, None, Kc, Vc, ops.rope_table(max_seq, hd, 1e4).cuda(), rows, nh, nkv,
                                 hd, pos0, max_seq, 1e-6, False, False)
    torch.cuda.synchronize()
    assert np.abs(Q.cpu().numpy() - want_q).max() <= 2e-6 * np.abs(want_q).max()
    assert np.abs(K.cpu().numpy() - want_k).max() <= 2e-6 * np.abs(want_k).max()
    assert np.array_equal(Kc[pos0:pos0 + rows].cpu().numpy(), K.cpu().numpy())


@pytest.mark.parametrize("kv_fp16", [True, False])
@pytest.mark.parametrize("nh,nkv,hd,pos0,rows", [(32, 8, 128, 0, 70), (32, 8, 128, 300, 17), (4, 2, 64, 0, 33),
                                                 (4, 4, 64, 19, 5), (16, 2, 128, 1, 1), (16, 2, 128, 3, 40),
                                                 (4, 4, 128, 0, 130), (8, 4, 64, 31, 97), (8, 1, 64, 0, 16),
                                                 (32, 8, 128, 1000, 64), (32, 8, 128, 15000, 33), (8, 4, 256, 100, 20),
                                                 (2, 1, 256, 0, 5), (28, 4, 128, 50, 20), (40, 8, 128, 0, 17), (12, 2, 64, 7, 33),
                                                 # chunks that end beyond position 512: two wave groups per workgroup
                                                 (8, 4, 64, 500, 70), (4, 4, 128, 480, 130), (16, 2, 128, 600, 40), (4, 4, 64, 0, 530),
                                                 # 3 / 5 / 6 / 7 query heads per kv head on the matrix cores (a row takes 4 or 8 head
                                                 # slots, the spare ones are computed and dropped): both wave-group counts, ragged rows
                                                 (24, 8, 64, 0, 100), (6, 2, 128, 700, 150), (20, 4, 128, 90, 257), (12, 2, 64, 520, 31),
                                                 (28, 4, 128, 1000, 200), (14, 2, 64, 0, 16),
                                                 # heads of 256 on the matrix cores (the output's head dimension split over two
                                                 # sets of waves): 1 / 2 / 4 / 3 query heads per kv head, ragged rows, long walks
                                                 (8, 4, 256, 0, 130), (4, 4, 256, 700, 67), (8, 2, 256, 33, 200), (6, 2, 256, 1200, 45),
                                                 (16, 4, 256, 0, 512)])
def test_prefill_attention_vs_oracle(dev, po, kv_fp16, nh, nkv, hd, pos0, rows):
    """Row r attends to cache positions [0, pos0 + r]: later rows of the same batch must not leak in.  With an
    fp16 cache and 16 or more rows the matrix-core kernel runs (Q and the softmax weights rounded to fp16: bar
    1e-3 of the output's maximum, measured 1.5e-4..2.8e-4); otherwise the fp32 kernel (bar 1e-4)."""
    T = pos0 + rows
    max_seq = T + 2
    kvd = nkv * hd
    r = synth.rng_for(64, nh, hd, pos0, rows)
    k16 = r.standard_normal((max_seq, kvd), dtype=np.float32).astype(np.float16)
    v16 = r.standard_normal((max_seq, kvd), dtype=np.float32).astype(np.float16)
    kf, vf = k16.astype(np.float32), v16.astype(np.float32)
    q = (r.standard_normal((rows, nh * hd), dtype=np.float32) * 0.5)
    scale = 1.0 / np.sqrt(hd)
    want = np.stack([np.concatenate([po.attn_head(q[m, h * hd:(h + 1) * hd], kf, vf, pos0 + m + 1, kvd, hd, scale,
                                                  col0=(h // (nh // nkv)) * hd) for h in range(nh)]) for m in range(rows)])
    dt = torch.float16 if kv_fp16 else torch.float32
    Kc, Vc = cu(kf).to(dt), cu(vf).to(dt)
    Kc[T:] = float("nan")
    Vc[T:] = float("nan")
    O = torch.full((rows, nh * hd), 9.0, device="cuda")
    ops.prefill_attention(cu(q), Kc, Vc, O, rows, nh, nkv, hd, pos0, max_seq, scale, kv_fp16)
    torch.cuda.synchronize()
    got = O.cpu().numpy()
    assert np.all(np.isfinite(got))
    e = np.abs(got - want).max() / np.abs(want).max()
    print("attention nh %d nkv %d hd %d pos0 %d rows %d fp16 %s: max err / max %.2e" % (nh, nkv, hd, pos0, rows, kv_fp16, e), flush=True)
    assert e <= (1e-3 if kv_fp16 and rows >= 16 else 1e-4)


def test_prefill_attention_rejects_bad_shapes(dev):
    z = torch.zeros(64 * 64, device="cuda")
    with pytest.raises(PtmError):
        ops.prefill_attention(z, z, z, z, 4, 4, 3, 64, 0, 16, 0.1, False)   # heads not a multiple of kv heads
    with pytest.raises(PtmError):
        ops.prefill_attention(z, z, z, z, 4, 4, 2, 96, 0, 16, 0.1, False)   # head size this path has no kernel for
    with pytest.raises(PtmError):
        ops.prefill_attention(z, z, z, z, 4, 4, 2, 64, 14, 16, 0.1, False)  # rows run past the cache


# ---- matmul on fp32 rows with accumulate -----------------------------------------------------------------------
@pytest.mark.parametrize("qt", [12, 14])
@pytest.mark.parametrize("M,K,N", [(70, 1024, 300),      # 2 column tiles, 4 super-blocks: K split in 2
                                   (33, 2560, 1024),     # k/v projection of Qwen3-4B: K split in 5
                                   (130, 4864, 2560),    # down-projection-like: 19 super-blocks in 6 uneven splits
                                   (5, 256, 48),         # one super-block: no split
                                   (64, 512, 9728)])     # wide: no split
def test_qgemm_f16_f32_rows_and_accumulate(dev, po, qt, M, K, N):
    r = synth.rng_for(65, qt, M, K, N)
    W = synth.make_weight(r, qt, N, K)
    x = r.standard_normal((M, K), dtype=np.float32)
    y0 = r.standard_normal((M, N), dtype=np.float32)
    ref = np.stack([po.gemv(qt, W, x[m]) for m in range(M)])
    ws = torch.empty(ops.qgemm_f16_f32_workspace_bytes(M, K, N), dtype=torch.uint8, device="cuda")
    Wd, Xd = cu(W), cu(x)
    Y = torch.full((M, N), 5.0, device="cuda")
    ops.matmul_q_f16_f32(qt, Wd, Xd, Y, M, K, N, W.shape[1], ws)
    Ya = cu(y0)
    ops.matmul_q_f16_f32(qt, Wd, Xd, Ya, M, K, N, W.shape[1], ws, accumulate=True)
    torch.cuda.synchronize()
    rms = np.sqrt((ref.astype(np.float64) ** 2).mean())
    assert np.abs(Y.cpu().numpy() - ref).max() / rms <= PREFILL_TOL
    assert np.array_equal(bits(Ya.cpu().numpy()), bits(y0 + Y.cpu().numpy()))   # Y += is one fp32 add of the same product
    # a row's result does not depend on how many rows share the launch, within a row class (the K split is a function
    # of N, K and of whether M is at most 128, at most 256, or more)
    m3 = min(3, M) if M <= 128 else 129
    Y3 = torch.empty((m3, N), device="cuda")
    ops.matmul_q_f16_f32(qt, Wd, Xd[:m3].contiguous(), Y3, m3, K, N, W.shape[1], ws)
    torch.cuda.synchronize()
    assert np.array_equal(bits(Y3.cpu().numpy()), bits(Y[:m3].cpu().numpy()))


# ---- whole prefill -------------------------------------------------------------------------------------------------
def build_tiny(seeds):
    cfg = dict(synth.TINY)
    layers = [synth.make_layer(seeds["tiny"], i, cfg) for i in range(cfg["n_layers"])]
    head = synth.make_head(seeds["tiny"], cfg)
    return cfg, layers, head


def logit_errors(got, want):
    sd = float(want.std())
    d = got.astype(np.float64) - want
    srt = np.sort(want)
    return float(np.abs(d).max()) / sd, float(np.sqrt((d ** 2).mean())) / sd, float(srt[-1] - srt[-2]) / sd


def check_logits(got, want, tok_g, tok_o, what):
    err, rms, margin = logit_errors(got, want)
    assert rms <= E2E_RMS_TOL and err <= E2E_MAX_TOL, (what, err, rms)
    if margin > 2 * err:
        assert tok_g == tok_o, (what, margin, err)
    return err, rms, margin


def row_errors(g, c):
    return np.sqrt(((g - c) ** 2).sum(axis=1) / (c ** 2).sum(axis=1))


def check_kv_rows(g, c, layer, what):
    """Cache rows the prefill appended against the oracle's.  Layer 0's rows are one GEMM deep.  Deeper rows carry
    the Q8 rounding noise of the layers before; a few positions of a random-weight model sit on a boundary where
    that noise tips the whole row (the oracle does the same against itself under a 5e-4 input perturbation), so the
    bar there is on the median row and on how many rows stray."""
    e = row_errors(g, c)
    print("  layer %d %s rows: rel err median %.2e worst %.2e" % (layer, what, np.median(e), e.max()), flush=True)
    if layer == 0:
        assert e.max() <= STAGE_TOL, (layer, what)
    else:
        assert np.median(e) <= 3 * E2E_RMS_TOL and int((e > 0.1).sum()) <= max(2, len(e) // 16), (layer, what)


def follow(dec, om, tok, steps):
    """Decode `steps` more tokens on both sides; the GPU reads the KV rows its prefill wrote."""
    for st in range(steps):
        tok_o = om.step(tok)
        tok_g = dec.step(tok)
        check_logits(dec.logits(), om.logits, tok_g, tok_o, ("follow", st))
        tok = tok_o  # keep both sides on the oracle's sequence


@pytest.mark.parametrize("kv_fp16", [True, False])
@pytest.mark.parametrize("pos0,n,chunk", [(0, 23, 0), (0, 23, 7), (19, 12, 5), (0, 1, 0)])
def test_tiny_prefill_vs_oracle_token_by_token(dev, po, seeds, kv_fp16, pos0, n, chunk):
    from prometorch_amd.decode import Decoder
    cfg, layers, head = build_tiny(seeds)
    om = po.OracleModel(cfg, layers, head, 64, kv_fp16=kv_fp16)
    dec = Decoder(cfg, layers, head, max_seq=64, kv_fp16=kv_fp16, use_graph=True)
    if pos0:
        for i in range(cfg["n_layers"]):
            k, v = synth.make_kv_prefill(seeds["tiny"], i, cfg, pos0)
            om.set_kv(i, k, v)
            dec.set_kv(i, k, v)
        dec.set_past_len(pos0)
    prompt = [int(t) for t in synth.rng_for(66, pos0, n).integers(0, cfg["vocab"], n)]
    for t in prompt:
        tok_o = om.step(t)
    tok_g = dec.prefill(prompt, chunk_rows=chunk)
    sd = float(om.logits.std())
    err = float(np.abs(dec.logits() - om.logits).max()) / sd
    srt = np.sort(om.logits)
    margin = float(srt[-1] - srt[-2]) / sd
    rms = float(np.sqrt(((dec.logits() - om.logits) ** 2).mean())) / sd
    print("prefill pos0 %d n %d chunk %d: logit err/std max %.2e rms %.2e, top-2 margin/std %.3f" % (pos0, n, chunk, err, rms, margin), flush=True)
    # appended K/V rows against the oracle's
    for li in range(cfg["n_layers"]):
        for nm, gpu_c, cpu_c in (("k", dec.k_cache[li], om.k_cache[li]), ("v", dec.v_cache[li], om.v_cache[li])):
            check_kv_rows(gpu_c[pos0:pos0 + n].float().cpu().numpy(), cpu_c[pos0:pos0 + n], li, nm)
    check_logits(dec.logits(), om.logits, tok_g, tok_o, "prefill")
    follow(dec, om, tok_o, 6)
    dec.close()


def test_prefill_layer_stage_by_stage_on_identical_inputs(dev, po, seeds):
    """One layer of the prompt path rebuilt from the C ABI's row-batched entry points in the order ptm_decode_prefill
    issues them; after every stage the oracle computes the same stage from the GPU's OWN input to it, so nothing
    compounds and each stage is held to STAGE_TOL."""
    cfg, layers, head = build_tiny(seeds)
    Ld = layers[0]
    H, nh, nkv, hd, I = cfg["hidden"], cfg["n_heads"], cfg["n_kv_heads"], cfg["head_dim"], cfg["inter"]
    qd, kvd, M, pos0, max_seq, eps = nh * hd, nkv * hd, 23, 9, 40, cfg["eps"]
    r = synth.rng_for(70)
    k0, v0 = synth.make_kv_prefill(seeds["tiny"], 0, cfg, pos0)
    Kc = torch.zeros(max_seq, kvd, dtype=torch.float16, device="cuda")
    Vc = torch.zeros(max_seq, kvd, dtype=torch.float16, device="cuda")
    Kc[:pos0], Vc[:pos0] = cu(k0), cu(v0)
    ws = torch.empty(max(ops.qgemm_f16_f32_workspace_bytes(M, k_, n_) for k_, n_ in ((H, qd), (H, kvd), (qd, H), (H, I), (I, H))),
                     dtype=torch.uint8, device="cuda")
    Wd = {n: cu(Ld[n][1]) for n in ("q", "k", "v", "o", "gate", "up", "down")}

    def gemm(name, X, Y, acc=False):
        qt, W = Ld[name]
        ops.matmul_q_f16_f32(qt, Wd[name], X, Y, M, X.shape[1], W.shape[0], W.shape[1], ws, accumulate=acc)

    def rows_close(got, want, what, tol=STAGE_TOL):
        e = np.abs(got - want).max() / np.sqrt((want.astype(np.float64) ** 2).mean())
        print("%-12s max err / rms %.2e" % (what, e), flush=True)
        assert e <= tol, what

    def cpu_gemm(name, X):
        qt, W = Ld[name]
        return np.stack([po.gemv(qt, W, X[m]) for m in range(M)])

    table = po.dequant(14, head["lm_head"]).reshape(cfg["vocab"], H)
    toks = r.integers(0, cfg["vocab"], M).astype(np.int32)
    X = torch.empty(M, H, device="cuda")
    ops.embedding_rows(None, cu(head["lm_head"]), head["lm_head"].shape[1], cu(toks), M, H, cfg["vocab"], X)
    x = X.cpu().numpy()
    assert np.array_equal(bits(x), bits(table[toks]))
    Xn = torch.empty(M, H, device="cuda")
    ops.launch_rms_norm(X, cu(Ld["attn_norm"]), Xn, M, H, eps, False)
    xn = Xn.cpu().numpy()
    rows_close(xn, np.stack([po.rmsnorm(x[m], Ld["attn_norm"], eps) for m in range(M)]), "attn_norm", 1e-5)
    Q, K, V = torch.empty(M, qd, device="cuda"), torch.empty(M, kvd, device="cuda"), torch.empty(M, kvd, device="cuda")
    gemm("q", Xn, Q), gemm("k", Xn, K), gemm("v", Xn, V)
    q, k, v = Q.cpu().numpy(), K.cpu().numpy(), V.cpu().numpy()
    rows_close(q, cpu_gemm("q", xn), "q proj")
    rows_close(k, cpu_gemm("k", xn), "k proj")
    rows_close(v, cpu_gemm("v", xn), "v proj")
    ops.qknorm_rope_kvwrite_rows(Q, K, V, cu(Ld["q_norm"]), cu(Ld["k_norm"]), Kc, Vc, ops.rope_table(max_seq, hd, cfg["rope_base"]).cuda(),
                                 M, nh, nkv, hd, pos0, max_seq, eps, False, True)
    want_q, want_k = np.empty_like(q), np.empty_like(k)
    for m in range(M):
        qn = np.concatenate([po.rmsnorm(q[m, h * hd:(h + 1) * hd], Ld["q_norm"], eps) for h in range(nh)])
        kn = np.concatenate([po.rmsnorm(k[m, h * hd:(h + 1) * hd], Ld["k_norm"], eps) for h in range(nkv)])
        c, s = po.rope_tables(pos0 + m, hd, cfg["rope_base"])
        want_q[m], want_k[m] = po.rope_neox(qn, kn, c, s, nh, nkv, hd)
    qr = Q.cpu().numpy()
    rows_close(qr, want_q, "q norm+rope", 1e-5)
    rows_close(K.cpu().numpy(), want_k, "k norm+rope", 1e-5)
    kf, vf = Kc.float().cpu().numpy(), Vc.float().cpu().numpy()
    A = torch.empty(M, qd, device="cuda")
    scale = 1.0 / np.sqrt(hd)
    ops.prefill_attention(Q, Kc, Vc, A, M, nh, nkv, hd, pos0, max_seq, scale, True)
    a = A.cpu().numpy()
    rows_close(a, np.stack([np.concatenate([po.attn_head(qr[m, h * hd:(h + 1) * hd], kf, vf, pos0 + m + 1, kvd, hd, scale,
                                                         col0=(h // (nh // nkv)) * hd) for h in range(nh)]) for m in range(M)]),
               "attention", STAGE_TOL)
    gemm("o", A, X, acc=True)
    x1 = X.cpu().numpy()
    rows_close(x1 - x, cpu_gemm("o", a), "o proj (+=)")
    ops.launch_rms_norm(X, cu(Ld["ffn_norm"]), Xn, M, H, eps, False)
    xn = Xn.cpu().numpy()
    rows_close(xn, np.stack([po.rmsnorm(x1[m], Ld["ffn_norm"], eps) for m in range(M)]), "ffn_norm", 1e-5)
    G, U = torch.empty(M, I, device="cuda"), torch.empty(M, I, device="cuda")
    gemm("gate", Xn, G), gemm("up", Xn, U)
    g, u = G.cpu().numpy(), U.cpu().numpy()
    rows_close(g, cpu_gemm("gate", xn), "gate proj")
    rows_close(u, cpu_gemm("up", xn), "up proj")
    ops.launch_silu_mul(G, U, G, M * I)
    act = G.cpu().numpy()
    rows_close(act, np.stack([po.silu_mul(g[m], u[m]) for m in range(M)]), "silu*up", 1e-5)
    gemm("down", G, X, acc=True)
    rows_close(X.cpu().numpy() - x1, cpu_gemm("down", act), "down proj (+=)")


def test_q8_rounding_noise_floor_of_the_oracle(po, seeds):
    """The yardstick for the end-to-end bars, CPU only: the oracle against ITSELF with its input embedding perturbed
    by 5e-4 relative (the size of the fp16 GEMM's error).  The Q8 activation rounding turns that into a logit
    difference of the same order as the one between the GPU prefill and the oracle."""
    cfg, layers, head = build_tiny(seeds)
    table = po.dequant(14, head["lm_head"]).reshape(cfg["vocab"], cfg["hidden"])
    noise = synth.rng_for(71).standard_normal(table.shape, dtype=np.float32)
    a = po.OracleModel(cfg, layers, head, 64, kv_fp16=True, embedding=table)
    b = po.OracleModel(cfg, layers, head, 64, kv_fp16=True, embedding=table * (1 + np.float32(5e-4) * noise))
    prompt = [int(t) for t in synth.rng_for(66, 0, 23).integers(0, cfg["vocab"], 23)]
    errs = []
    for t in prompt:
        a.step(t)
        b.step(t)
        errs.append(logit_errors(b.logits, a.logits)[:2])
    mx, rms = np.median(np.asarray(errs), axis=0)   # medians: single steps of the tiny model can be far more sensitive
    print("oracle vs perturbed oracle over %d steps: median logit err/std max %.2e rms %.2e" % (len(errs), mx, rms), flush=True)
    assert 2e-3 <= rms <= E2E_RMS_TOL and 1e-2 <= mx <= E2E_MAX_TOL


def test_prefill_chunking_does_not_change_the_result(dev, seeds):
    """Chunks only bound the scratch: rows are independent in every GEMM (the K split depends on N, K and the row class,
    here always "at most 128 rows") and
    attention reads the cache in the same tiles, so any chunk size that stays on the same attention kernel gives
    bit-identical logits; chunks under 16 rows use the fp32 attention kernel and agree within the end-to-end bars."""
    from prometorch_amd.decode import Decoder
    cfg, layers, head = build_tiny(seeds)
    prompt = [int(t) for t in synth.rng_for(67).integers(0, cfg["vocab"], 48)]
    outs = []
    for chunk in (0, 16, 24, 3):
        dec = Decoder(cfg, layers, head, max_seq=64, kv_fp16=True, use_graph=False)
        tok = dec.prefill(prompt, chunk_rows=chunk)
        outs.append((tok, dec.logits()))
        dec.close()
    for tok, lg in outs[1:3]:
        assert tok == outs[0][0] and np.array_equal(bits(lg), bits(outs[0][1]))
    err, rms, margin = logit_errors(outs[3][1], outs[0][1])
    assert rms <= E2E_RMS_TOL and err <= E2E_MAX_TOL
    if margin > 2 * err:
        assert outs[3][0] == outs[0][0]


def test_reserved_prefill_allocates_nothing_and_changes_nothing(dev, seeds):
    """ptm_decode_reserve_prefill sizes the row scratch ahead of time: a prefill of at most that many rows then leaves the
    amount of free device memory untouched (no allocation after set-up), with logits bit-identical to a decoder that allocates
    on first use; a longer prompt afterwards still works (the scratch grows)."""
    from prometorch_amd.decode import Decoder
    from prometorch_amd._lib import check
    cfg, layers, head = build_tiny(seeds)
    prompt = [int(t) for t in synth.rng_for(69).integers(0, cfg["vocab"], 40)]
    plain = Decoder(cfg, layers, head, max_seq=96, kv_fp16=True, use_graph=False)
    t_plain = plain.prefill(prompt)
    lg_plain = plain.logits()
    plain.close()
    dec = Decoder(cfg, layers, head, max_seq=96, kv_fp16=True, use_graph=False)
    check(dec.L.ptm_decode_reserve_prefill(dec.h, 48), "reserve_prefill")
    torch.cuda.synchronize()
    free_before = torch.cuda.mem_get_info()[0]
    tok = dec.prefill(prompt)
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info()[0] == free_before
    assert tok == t_plain and np.array_equal(bits(dec.logits()), bits(lg_plain))
    more = [int(t) for t in synth.rng_for(70).integers(0, cfg["vocab"], 50)]
    dec.prefill(more)                                   # beyond the reservation: allowed, allocates
    assert dec.L.ptm_decode_reserve_prefill(dec.h, 0) < 0   # a reservation of no rows is an error
    dec.close()


def test_prefill_then_prefill_continues_the_context(dev, po, seeds):
    """Two prefills in a row (a second user turn) equal one prefill of the concatenation."""
    from prometorch_amd.decode import Decoder
    cfg, layers, head = build_tiny(seeds)
    prompt = [int(t) for t in synth.rng_for(68).integers(0, cfg["vocab"], 30)]
    a = Decoder(cfg, layers, head, max_seq=64, kv_fp16=True, use_graph=True)
    b = Decoder(cfg, layers, head, max_seq=64, kv_fp16=True, use_graph=True)
    ta = a.prefill(prompt)
    b.prefill(prompt[:11])
    b.step(prompt[11])                 # a decode step in between is the same as a one-row prefill
    tb = b.prefill(prompt[12:])
    err, rms, margin = logit_errors(b.logits(), a.logits())
    assert rms <= E2E_RMS_TOL and err <= E2E_MAX_TOL
    if margin > 2 * err:
        assert ta == tb
    a.close()
    b.close()


def test_prefill_argument_errors(dev, seeds):
    from prometorch_amd.decode import Decoder
    cfg, layers, head = build_tiny(seeds)
    dec = Decoder(cfg, layers, head, max_seq=32, kv_fp16=True, use_graph=False)
    with pytest.raises(PtmError):
        dec.prefill([1] * 33)                     # longer than the cache
    with pytest.raises(PtmError):
        dec.prefill([1, cfg["vocab"], 2])         # token id outside the table
    with pytest.raises(PtmError):
        dec.prefill([])                           # empty prompt
    assert dec.prefill([1] * 32) >= 0             # exactly fills the cache
    with pytest.raises(PtmError):
        dec.prefill([1])                          # no room left
    dec.close()


def test_qwen3_4b_shape_prefill_64_tokens(dev, po, seeds):
    """Full-size layers (36 x Qwen3-4B shapes, Q4_K_M mix): a 64-token prompt in two chunks against the oracle
    stepping it token by token, then eight decode steps that read the prefilled cache."""
    from prometorch_amd.decode import Decoder
    cfg = dict(synth.QWEN3_4B)
    seed = seeds["cfg4"]
    layers = [synth.make_layer(seed, i, cfg) for i in range(cfg["n_layers"])]
    head = synth.make_head(seed, cfg)
    om = po.OracleModel(cfg, layers, head, 128, kv_fp16=True)
    dec = Decoder(cfg, layers, head, max_seq=128, kv_fp16=True, use_graph=True)
    prompt = [int(t) for t in synth.rng_for(69).integers(0, cfg["vocab"], 64)]
    for t in prompt:
        tok_o = om.step(t)
    tok_g = dec.prefill(prompt, chunk_rows=48)
    err, rms, margin = check_logits(dec.logits(), om.logits, tok_g, tok_o, "prefill")
    print("qwen3-4b prefill 64: logit err/std max %.2e rms %.2e, top-2 margin/std %.3f, tokens %d/%d" % (err, rms, margin, tok_g, tok_o), flush=True)
    for li in (0, 17, 35):
        check_kv_rows(dec.k_cache[li][:64].float().cpu().numpy(), om.k_cache[li][:64], li, "k")
        check_kv_rows(dec.v_cache[li][:64].float().cpu().numpy(), om.v_cache[li][:64], li, "v")
    follow(dec, om, tok_o, 8)
    dec.close()


@pytest.mark.parametrize("n,chunk", [(1100, 512), (1100, 0)])
def test_long_prompt_prefill_vs_oracle(dev, po, seeds, n, chunk):
    """The row classes of real prompts (257..1024 rows and more than 1024; gate and up in one launch; two wave groups in the
    attention; chunks that continue a filled cache) against the ORACLE, not only against this decoder's own stepping: three
    full-width Qwen3-4B layers, an 1100-token prompt, the oracle fed token by token (1100 steps of 3 layers on the CPU).
    Logits at five prompt lengths, greedy token where the margin allows, cache rows of every layer."""
    from prometorch_amd.decode import Decoder
    cfg = dict(synth.QWEN3_4B)
    cfg["n_layers"] = 3
    seed = seeds["cfg4"]
    layers = [synth.make_layer(seed, i, cfg) for i in range(3)]
    head = synth.make_head(seed, cfg)
    om = po.OracleModel(cfg, layers, head, n + 16, kv_fp16=True)
    dec = Decoder(cfg, layers, head, max_seq=n + 16, kv_fp16=True, use_graph=True)
    prompt = [int(t) for t in synth.rng_for(70, n).integers(0, cfg["vocab"], n)]
    ends = list(range(n - 4, n + 1))
    want, want_tok = {}, {}
    for i, t in enumerate(prompt):
        tok_o = om.step(t)
        if i + 1 in ends:
            want[i + 1], want_tok[i + 1] = om.logits.copy(), tok_o
    # A random-weight model amplifies the int8 rounding noise of single positions (the oracle does the same against itself
    # under a 5e-4 input perturbation, test_q8_rounding_noise_floor_of_the_oracle), so the logits are compared at five prompt
    # lengths: the bar of the whole-model comparison on their median, no length far off
    rmss, errs = [], []
    for e in ends:
        dec.set_past_len(0)
        tok_g = dec.prefill(prompt[:e], chunk_rows=chunk)
        err, rms, margin = logit_errors(dec.logits(), want[e])
        rmss.append(rms)
        errs.append(err)
        if margin > 2 * err:
            assert tok_g == want_tok[e], (e, margin, err)
    print("prefill %d tokens chunk %d vs oracle: logit rms err/std at 5 lengths %s, max %s" %
          (n, chunk, ["%.1e" % r for r in rmss], ["%.1e" % r for r in errs]), flush=True)
    assert np.median(rmss) <= E2E_RMS_TOL and max(rmss) <= LONG_RMS_WORST, rmss
    for li in range(3):   # the cache as the last (full-length) prefill left it
        check_kv_rows(dec.k_cache[li][:n].float().cpu().numpy(), om.k_cache[li][:n], li, "k")
        check_kv_rows(dec.v_cache[li][:n].float().cpu().numpy(), om.v_cache[li][:n], li, "v")
    dec.close()


@pytest.mark.parametrize("n,chunk", [(1100, 0), (1100, 512), (1100, 1024), (1100, 300), (2048, 0)])
def test_long_prompt_prefill_matches_token_by_token_decode(dev, seeds, n, chunk):
    """The row classes real prompts run in (257..1024 rows, more than 1024; gate and up in one launch; two wave groups in
    the attention): three full-width Qwen3-4B layers, the prompt prefilled in chunks of that size against the same decoder
    fed one token at a time (the decode step is pinned against the oracle elsewhere).  Size-independent property:
    prefill and stepping compute the same function.  A random-weight model amplifies the Q8 rounding noise of single
    positions (see check_kv_rows), so the logits are compared at five prompt lengths and the bar is on their median, with
    no length allowed to be far off."""
    from prometorch_amd.decode import Decoder
    cfg = dict(synth.QWEN3_4B)
    cfg["n_layers"] = 3
    seed = seeds["cfg4"]
    layers = [synth.make_layer(seed, i, cfg) for i in range(3)]
    head = synth.make_head(seed, cfg)
    dec = Decoder(cfg, layers, head, max_seq=n + 16, kv_fp16=True, use_graph=True)
    prompt = [int(t) for t in synth.rng_for(70, n).integers(0, cfg["vocab"], n)]
    ends = list(range(n - 4, n + 1))
    want, want_tok = {}, {}
    for i, t in enumerate(prompt):
        tok = dec.step(t)
        if i + 1 in ends:
            want[i + 1], want_tok[i + 1] = dec.logits().copy(), tok
    want_k = [dec.k_cache[li][:n].float().cpu().numpy() for li in range(3)]
    want_v = [dec.v_cache[li][:n].float().cpu().numpy() for li in range(3)]
    rmss = []
    for e in ends:
        dec.set_past_len(0)
        tok_p = dec.prefill(prompt[:e], chunk_rows=chunk)
        err, rms, margin = logit_errors(dec.logits(), want[e])
        rmss.append(rms)
        if margin > 2 * err:
            assert tok_p == want_tok[e], (e, margin, err)
    print("prefill %d tokens chunk %d vs stepping: logit rms err/std at 5 lengths %s" % (n, chunk, ["%.1e" % r for r in rmss]), flush=True)
    assert np.median(rmss) <= E2E_RMS_TOL and max(rmss) <= LONG_RMS_WORST, rmss
    for li in range(3):  # the cache as the last (full-length) prefill left it
        check_kv_rows(dec.k_cache[li][:n].float().cpu().numpy(), want_k[li], li, "k")
        check_kv_rows(dec.v_cache[li][:n].float().cpu().numpy(), want_v[li], li, "v")
    dec.close()


def test_qgemm_f16_random_shapes_vs_oracle(dev, po):
    """A fixed pseudo-random sweep of the fast prefill GEMM over row counts (both tile heights, ragged last tiles),
    widths and lengths (split and unsplit K), both weight types, against the oracle's row-by-row GEMVs."""
    r = np.random.default_rng(20251126)
    worst = 0.0
    for case in range(12):
        qt = int(r.choice([12, 14]))
        M = int(r.integers(1, 400)) if case % 3 else int(r.choice([1, 64, 65, 128, 129, 256, 257]))
        K = int(r.integers(1, 17)) * 256
        N = int(r.integers(1, 1600))
        rr = synth.rng_for(72, case)
        W = synth.make_weight(rr, qt, N, K)
        x = rr.standard_normal((M, K), dtype=np.float32)
        ref = np.stack([po.gemv(qt, W, x[m]) for m in range(M)])
        ws = torch.empty(ops.qgemm_f16_f32_workspace_bytes(M, K, N), dtype=torch.uint8, device="cuda")
        Y = torch.full((M, N), -3.0, device="cuda")
        ops.matmul_q_f16_f32(qt, cu(W), cu(x), Y, M, K, N, W.shape[1], ws)
        torch.cuda.synchronize()
        e = float(np.abs(Y.cpu().numpy() - ref).max() / np.sqrt((ref.astype(np.float64) ** 2).mean()))
        worst = max(worst, e)
        assert e <= PREFILL_TOL, (case, qt, M, K, N, e)
    print("worst error / rms(y): %.2e" % worst)
