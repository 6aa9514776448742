"""CPU: the oracle (oracle/ptm_oracle.c) against the golden vectors written by the compiled
reference, and against what the mathematics fixes independently (numpy closed forms, float64,
exact integer arithmetic).  No GPU."""
import numpy as np
import pytest

from conftest import bits, sha, sha_of
from prometorch_amd.testing import synth


def test_fp16_all_values_vs_numpy_and_reference(po, golden):
    h = np.arange(65536, dtype=np.uint16)
    mine = np.array([po.fp16_to_fp32(int(v)) for v in h], np.float32)
    want = h.view(np.float16).astype(np.float32)
    nan = np.isnan(want)
    assert np.array_equal(bits(mine)[~nan], bits(want)[~nan])
    assert np.all(np.isnan(mine[nan]))
    assert sha(mine) == sha_of(golden, "fp16_table_sha")  # includes the reference's NaN payloads


def test_fp32_to_fp16_rne(po):
    rng = synth.rng_for(5)
    x = np.concatenate([rng.standard_normal(4096).astype(np.float32) * 100, np.array([0, -0.0, 65504, 65520, 1e-8, 6e-8], np.float32)])
    mine = np.array([po.lib().po_fp32_to_fp16(float(v)) for v in x], np.uint16)
    assert np.array_equal(mine, x.astype(np.float16).view(np.uint16))


def test_scale_min_pack_roundtrip_exhaustive(po):
    # every (scale, min) value in every slot: unpack(pack(v)) == v, against the oracle's C unpacker
    import ctypes as C
    for val in range(64):
        sc = np.full((1, 8), val, np.uint8)
        mn = np.full((1, 8), 63 - val, np.uint8)
        sc[0, val % 8] = (val * 7) % 64
        q12 = synth.pack_scales_k4(sc, mn)
        s2, m2 = synth.unpack_scales_k4(q12)
        assert np.array_equal(s2, sc) and np.array_equal(m2, mn)
        for j in range(8):
            a, b = C.c_uint8(), C.c_uint8()
            po.lib().po_get_scale_min_k4(j, po._p(q12), C.byref(a), C.byref(b))
            assert (a.value, b.value) == (sc[0, j], mn[0, j])
    rng = synth.rng_for(6)
    q12 = rng.integers(0, 256, size=(2000, 12), dtype=np.uint8)
    s, m = synth.unpack_scales_k4(q12)
    assert np.array_equal(synth.pack_scales_k4(s, m), q12)  # pack is the exact inverse on all 96 bits


@pytest.mark.parametrize("qt,key", [(12, "q4k"), (14, "q6k")])
def test_dequant_bit_exact_vs_reference_and_numpy(po, golden, qt, key):
    raw = golden[key + "_blocks"]
    want = golden[key + "_deq"]
    assert np.array_equal(bits(po.dequant(qt, raw)), bits(want))
    closed = synth.dequant_q4k_np(raw) if qt == 12 else synth.dequant_q6k_np(raw)
    assert np.array_equal(bits(closed), bits(want))


def test_q8_quantizer_vs_reference_and_invariants(po, golden):
    x = golden["q8_x"]
    d, s, q = po.quantize_x_q8(x)
    assert np.array_equal(bits(d), bits(golden["q8_d"]))
    assert np.array_equal(bits(s), bits(golden["q8_sum"]))
    assert np.array_equal(q, golden["q8_qs"])
    # invariants from the definition, in numpy: d = amax/127, q = clamp(rint(x * (1/d)))
    xb = x.reshape(-1, 32)
    amax = np.abs(xb).max(axis=1)
    dn = (amax / np.float32(127.0)).astype(np.float32)
    idn = np.where(dn > 0, np.float32(1.0) / np.where(dn > 0, dn, 1), np.float32(0)).astype(np.float32)
    qn = np.clip(np.rint((xb * idn[:, None]).astype(np.float32)), -127, 127).astype(np.int8)
    assert np.array_equal(qn.reshape(-1), q) and np.array_equal(bits(dn), bits(d))
    assert np.all(q.reshape(-1, 32)[1] == 0) and d[1] == 0  # all-zero block
    assert list(q[64:70]) == [127, 0, 2, 2, 0, -2]          # ties go to even


def test_q4k_integer_dots_exact(po):
    rng = synth.rng_for(8)
    W = synth.make_q4k(rng, 4, 1024)
    x = synth.make_x(rng, 1024)
    _, _, q = po.quantize_x_q8(x)
    for r in range(4):
        isum = po.q4k_row_isums(W[r], q)
        blk = W[r].reshape(-1, 144)[:, 16:].reshape(-1, 4, 32)
        nib = np.stack([blk & 15, blk >> 4], axis=2).reshape(-1, 32).astype(np.int64)
        want = (nib * q.reshape(-1, 32).astype(np.int64)).sum(axis=1)
        assert np.array_equal(isum.astype(np.int64), want)


def test_q4k_gemv_cfg1_vs_reference(po, golden, seeds):
    r = synth.rng_for(seeds["cfg1"])
    W = synth.make_q4k(r, 9728, 2560)
    x = synth.make_x(r, 2560)
    y = po.gemv(12, W, x)
    assert np.array_equal(bits(y[:256]), bits(golden["cfg1_y256"]))
    assert sha(y) == sha_of(golden, "cfg1_sha")
    # the Q8-activation result is a perturbation of exact fp32-activation math, not something else
    yf = po.gemv(12, W, x, "f32")
    rms = np.sqrt((yf.astype(np.float64) ** 2).mean())
    assert np.abs(y - yf).max() / rms < 5e-2
    deq = po.dequant(12, W[:64]).reshape(64, 2560).astype(np.float64)
    assert np.abs(deq @ x.astype(np.float64) - yf[:64]).max() / rms < 1e-5


def test_gemv_ragged_shapes_vs_reference(po, golden, seeds):
    rr = synth.rng_for(seeds["ragged"])
    for i, (qt, N, K) in enumerate([(12, 33, 512), (12, 1, 256), (12, 77, 2560), (14, 7, 256), (14, 45, 1024)]):
        W = synth.make_weight(rr, qt, N, K)
        x = synth.make_x(rr, K)
        assert np.array_equal(bits(po.gemv(qt, W, x)), bits(golden[f"ragged{i}_y"])), (qt, N, K)


def test_q6k_gemv_vs_reference_and_float64(po, golden, seeds):
    L = synth.make_layer(seeds["cfg3"], 0, synth.QWEN3_4B)
    for i, (name, qt) in enumerate(synth.LAYER_MATS):
        _, W = L[name]
        K = W.shape[1] // (144 if qt == 12 else 210) * 256
        x = synth.make_x(synth.rng_for(seeds["cfg3"], 5, i), K)
        y = po.gemv(qt, W, x)
        assert sha(y) == sha_of(golden, f"cfg3_{name}_sha"), name
        assert np.array_equal(bits(y[:: max(1, y.size // 64)][:64]), bits(golden[f"cfg3_{name}_y64"]))
        if qt == 14:
            deq = po.dequant(14, W[:32]).reshape(32, K).astype(np.float64)
            want = deq @ x.astype(np.float64)
            assert np.abs(y[:32] - want).max() / np.sqrt((want ** 2).mean()) < 1e-5


def test_dispatcher_unknown_type_is_noop(po):
    y = np.full(4, 7.0, np.float32)
    po.lib().po_cpu_quant_gemv(99, None, None, po._p(y), 256, 4, 144)
    assert np.all(y == 7.0)


def test_rmsnorm_vs_reference_and_float64(po, golden):
    out = po.rmsnorm(golden["rms_x"], golden["rms_g"], 1e-6)
    assert np.array_equal(bits(out), bits(golden["rms_out"]))
    x = golden["rms_x"].astype(np.float64)
    want = x / np.sqrt((x * x).mean() + 1e-6) * golden["rms_g"]
    assert np.abs(out - want).max() < 1e-5
    seq = po.rmsnorm(golden["rms_x"], golden["rms_g"], 1e-6, seq=True)
    assert np.abs(seq - want).max() < 1e-5


def test_rope_vs_reference_and_closed_form(po, golden):
    for pos in (0, 1, 2048, 2175):
        c, s = po.rope_tables(pos, 128, 1e6)
        assert np.array_equal(bits(c), bits(golden[f"rope_cos_{pos}"]))
        assert np.array_equal(bits(s), bits(golden[f"rope_sin_{pos}"]))
        d = np.arange(64, dtype=np.float64)
        th = pos * 1e6 ** (-2 * d / 128)
        assert np.abs(c - np.cos(th)).max() < 2e-4 and np.abs(s - np.sin(th)).max() < 2e-4  # fp32 theta
    c, s = golden["rope_cos_2048"], golden["rope_sin_2048"]
    q, k = po.rope_neox(golden["rope_q_in"], golden["rope_k_in"], c, s, 32, 8, 128)
    assert np.array_equal(bits(q), bits(golden["rope_q_out"]))
    assert np.array_equal(bits(k), bits(golden["rope_k_out"]))
    # NeoX pairing (d, d+64) and rotation direction, in float64
    qi = golden["rope_q_in"].reshape(32, 128).astype(np.float64)
    want = np.concatenate([qi[:, :64] * c - qi[:, 64:] * s, qi[:, :64] * s + qi[:, 64:] * c], axis=1)
    assert np.abs(q.reshape(32, 128) - want).max() < 1e-5
    assert np.allclose((q.reshape(32, 128) ** 2).sum(1), (qi ** 2).sum(1), rtol=1e-5)  # a rotation keeps norms


def test_exp_vs_reference_and_float64(po, golden):
    out = po.exp256(golden["exp_in"])
    assert np.array_equal(bits(out), bits(golden["exp_out"]))
    x = golden["exp_in"].astype(np.float64)
    ok = x > -87.0  # below that 2^n leaves the normal range and the routine returns 0 (or -inf)
    assert np.abs(out[ok] / np.exp(x[ok]) - 1).max() < 3e-7


def test_attention_head_vs_float64(po):
    rng = synth.rng_for(9)
    T, kvd, hd = 77, 256, 128
    q = synth.make_x(rng, hd)
    kc = rng.standard_normal((80, kvd), dtype=np.float32)
    vc = rng.standard_normal((80, kvd), dtype=np.float32)
    out = po.attn_head(q, kc, vc, T, kvd, hd, 1 / np.sqrt(hd), col0=128)
    s = (kc[:T, 128:].astype(np.float64) @ q.astype(np.float64)) / np.sqrt(hd)
    p = np.exp(s - s.max())
    want = (p / p.sum()) @ vc[:T, 128:].astype(np.float64)
    assert np.abs(out - want).max() < 1e-5


def test_silu_and_argmax(po):
    rng = synth.rng_for(10)
    g = (synth.make_x(rng, 1003) * 30).astype(np.float32)
    u = synth.make_x(rng, 1003)
    out = po.silu_mul(g, u)
    g64 = g.astype(np.float64)
    want = g64 / (1 + np.exp(-g64)) * u
    assert np.abs(out - want).max() <= 1e-5 * np.abs(want).max()
    x = synth.make_x(rng, 5000)
    assert po.argmax(x) == int(np.argmax(x))
    x[[17, 400, 4999]] = 99.0
    assert po.argmax(x) == 17  # lowest index wins a tie


def test_tiny_decode_bit_exact_vs_reference(po, golden, seeds):
    cfg = dict(synth.TINY)
    layers = [synth.make_layer(seeds["tiny"], i, cfg) for i in range(cfg["n_layers"])]
    head = synth.make_head(seeds["tiny"], cfg)
    om = po.OracleModel(cfg, layers, head, 64, kv_fp16=False)
    for i in range(cfg["n_layers"]):
        k, v = synth.make_kv_prefill(seeds["tiny"], i, cfg, 19)
        om.set_kv(i, k, v)
    tok = 3
    for st in range(12):
        tok = om.step(tok)
        assert tok == int(golden["tiny_tokens"][st])
        assert np.array_equal(bits(om.logits), bits(golden["tiny_logits"][st])), st


def test_llama_style_decode_and_rope_match_the_reference(po, seeds):
    """No QK-norm + interleaved rotation pairs (llama / mistral): oracle bit-identical to the compiled reference's
    forward_decode_cpu and rope_apply_fused (golden_llama.npz), and the rotation against float64."""
    import os
    from prometorch_amd.testing import synth
    g = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "golden_llama.npz"))
    cfg, layers, head = synth.tiny_llama(seeds["tiny"])
    om = po.OracleModel(cfg, layers, head, 64, kv_fp16=False)
    for i in range(cfg["n_layers"]):
        k, v = synth.make_kv_prefill(seeds["tiny"], i, cfg, 19)
        om.set_kv(i, k, v)
    tok = 3
    for st in range(12):
        tok = om.step(tok)
        assert tok == int(g["tokens"][st])
        assert np.array_equal(om.logits.view(np.uint32), g["logits"][st].view(np.uint32)), st
    r = synth.rng_for(seeds["blocks"], 77)
    q = (3 * r.standard_normal(32 * 128, dtype=np.float32)).astype(np.float32)
    k = (3 * r.standard_normal(8 * 128, dtype=np.float32)).astype(np.float32)
    c, s = po.rope_tables(2049, 128, 5.0e5)
    qr, kr = po.rope_norm(q, k, c, s, 32, 8, 128)
    assert np.array_equal(qr.view(np.uint32), g["rope_norm_q"].view(np.uint32))
    assert np.array_equal(kr.view(np.uint32), g["rope_norm_k"].view(np.uint32))
    # float64: pairs (2d, 2d+1) rotate by theta_d = pos * base^(-2d/hd)
    th = 2049.0 * 5.0e5 ** (-np.arange(64) / 64.0)
    q64 = q.astype(np.float64).reshape(32, 64, 2)
    want = np.stack([q64[..., 0] * np.cos(th) - q64[..., 1] * np.sin(th), q64[..., 0] * np.sin(th) + q64[..., 1] * np.cos(th)], -1)
    assert np.abs(qr.reshape(32, 64, 2) - want).max() <= 2e-3 * np.abs(want).max()   # fp32 angles of ~2e3 rad
    # linear position scaling: theta = (pos / scale) * freq -- table and a 12-step run at scale 4 against the reference's
    c4, s4 = po.rope_tables(2049, 128, 5.0e5, 4.0)
    assert np.array_equal(c4.view(np.uint32), g["scaled_cos"].view(np.uint32))
    assert np.array_equal(s4.view(np.uint32), g["scaled_sin"].view(np.uint32))
    th4 = (2049.0 / 4.0) * 5.0e5 ** (-np.arange(64) / 64.0)
    assert np.abs(c4 - np.cos(th4)).max() <= 1e-3 and np.abs(s4 - np.sin(th4)).max() <= 1e-3
    om = po.OracleModel(dict(cfg, rope_scale=4.0), layers, head, 64, kv_fp16=False)
    for i in range(cfg["n_layers"]):
        k, v = synth.make_kv_prefill(seeds["tiny"], i, cfg, 19)
        om.set_kv(i, k, v)
    tok = 3
    for st in range(12):
        tok = om.step(tok)
        assert tok == int(g["scaled_tokens"][st])
        assert np.array_equal(om.logits.view(np.uint32), g["scaled_logits"][st].view(np.uint32)), st
    assert np.abs(g["scaled_logits"][0] - g["logits"][0]).max() > g["logits"][0].std()   # the scale is not a no-op


def test_qwen2_style_biases_match_the_reference(po, seeds):
    """q / k / v bias vectors, no QK-norm, NeoX rotation (qwen2): oracle bit-identical to the compiled reference's
    forward_decode_cpu (golden_qwen2.npz); with any one of the three vectors zeroed the logits differ, so the golden run
    does exercise each of them."""
    import os
    from prometorch_amd.testing import synth
    g = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "golden_qwen2.npz"))
    cfg, layers, head = synth.tiny_qwen2(seeds["tiny"])

    def run(layers, steps):
        om = po.OracleModel(cfg, layers, head, 64, kv_fp16=False)
        for i in range(cfg["n_layers"]):
            k, v = synth.make_kv_prefill(seeds["tiny"], i, cfg, 19)
            om.set_kv(i, k, v)
        tok, toks, lg = 3, [], []
        for _ in range(steps):
            tok = om.step(tok)
            toks.append(tok)
            lg.append(om.logits.copy())
        return toks, np.stack(lg)

    toks, lg = run(layers, 12)
    assert toks == [int(t) for t in g["tokens"]]
    assert np.array_equal(lg.view(np.uint32), g["logits"].view(np.uint32))
    sigma = float(g["logits"][0].std())
    for drop in ("q_bias", "k_bias", "v_bias"):
        alt = [dict(L) for L in layers]
        for L in alt:
            L[drop] = np.zeros_like(L[drop])
        _, l1 = run(alt, 1)
        assert np.abs(l1[0] - g["logits"][0]).max() > 1e-2 * sigma, drop


def test_gemma_style_decode_matches_the_reference(po, seeds):
    """Scaled embeddings, tanh-GELU gate, post-norms, sliding-window layers with their own rotation base and linear
    position scaling on the global ones (gemma3): oracle bit-identical to the compiled reference's forward_decode_cpu
    (golden_gemma.npz); switching any one of the features off moves the first step's logits, so the run exercises each."""
    import os
    from prometorch_amd.testing import synth
    g = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "golden_gemma.npz"))
    cfg, layers, head = synth.tiny_gemma(seeds["tiny"])

    def run(cfg, layers, steps):
        om = po.OracleModel(cfg, layers, head, 64, kv_fp16=False)
        for i in range(cfg["n_layers"]):
            k, v = synth.make_kv_prefill(seeds["tiny"], i, cfg, 19)
            om.set_kv(i, k, v)
        tok, toks, lg = 3, [], []
        for _ in range(steps):
            tok = om.step(tok)
            toks.append(tok)
            lg.append(om.logits.copy())
        return toks, np.stack(lg)

    toks, lg = run(cfg, layers, 16)
    assert toks == [int(t) for t in g["tokens"]]
    assert np.array_equal(lg.view(np.uint32), g["logits"].view(np.uint32))
    sigma = float(g["logits"][0].std())
    for key, off in (("scale_embeddings", False), ("ffn_gelu", False), ("swa_window", 0), ("rope_swa_base", 1.0e6), ("rope_scale", 1.0)):
        _, l1 = run(dict(cfg, **{key: off}), layers, 1)
        assert np.abs(l1[0] - g["logits"][0]).max() > 1e-2 * sigma, key
    for name in ("post_attn_norm", "post_ffn_norm"):
        _, l1 = run(cfg, [{k: v for k, v in L.items() if k != name} for L in layers], 1)
        assert np.abs(l1[0] - g["logits"][0]).max() > 1e-2 * sigma, name


@pytest.mark.parametrize("family", ["llama", "qwen2", "gemma"])
def test_teacher_forced_family_runs_match_the_reference(po, seeds, family):
    """The greedy runs of the tiny family models settle on one token (llama: 999 x 12); these runs feed 16 distinct seeded ids
    instead, so every step reads another embedding row and appends other cache rows: oracle logits bit-identical to the
    compiled reference's forward_decode_cpu (forced_* of golden_<family>.npz), argmax identical."""
    import os
    from prometorch_amd.testing import synth
    g = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "golden_%s.npz" % family))
    cfg, layers, head = getattr(synth, "tiny_" + family)(seeds["tiny"])
    om = po.OracleModel(cfg, layers, head, 64, kv_fp16=False)
    for i in range(cfg["n_layers"]):
        om.set_kv(i, *synth.make_kv_prefill(seeds["tiny"], i, cfg, 19))
    feed = [int(t) for t in g["forced_feed"]]
    assert len(set(feed)) == 16
    for st, t in enumerate(feed):
        assert om.step(t) == int(g["forced_tokens"][st]), st
        assert np.array_equal(om.logits.view(np.uint32), g["forced_logits"][st].view(np.uint32)), st
    assert len(set(int(t) for t in g["forced_tokens"])) >= 9    # the outputs vary too


@pytest.mark.parametrize("seed", range(10))
def test_random_architectures_match_the_reference(po, seed):
    """synth.random_model draws every architectural switch at random (head width, heads per kv head, QK-norm, rotation
    pairing and scaling, biases, scaled embeddings, GELU, post-norms, sliding windows, per-matrix types): the oracle's
    logits over 4 steps are bit-identical to the compiled reference's (golden_random_arch.npz), so the switches are
    pinned in combination, not only one at a time."""
    import os
    from prometorch_amd.testing import synth
    g = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "golden_random_arch.npz"))
    cfg, layers, head = synth.random_model(seed)
    om = po.OracleModel(cfg, layers, head, 32, kv_fp16=False)
    for i in range(cfg["n_layers"]):
        k, v = synth.make_kv_prefill(1000 + seed, i, cfg, 11)
        om.set_kv(i, k, v)
    tok = 5
    for st in range(4):
        tok = om.step(tok)
        assert np.array_equal(om.logits.view(np.uint32), g["logits_%d" % seed][st].view(np.uint32)), st


def test_gelu_gate_against_float64(po):
    r = np.random.default_rng(3)
    gate = (3 * r.standard_normal(4096)).astype(np.float32)
    up = r.standard_normal(4096).astype(np.float32)
    got = gate.copy()
    po.lib().po_gelu_mul.argtypes = [po._vp, po._vp, po._i64]
    po.lib().po_gelu_mul(po._p(got), po._p(up), got.size)
    g64 = gate.astype(np.float64)
    want = 0.5 * g64 * (1 + np.tanh(np.sqrt(2 / np.pi) * (g64 + 0.044715 * g64 ** 3))) * up
    assert np.abs(got - want).max() <= 1e-5 * np.abs(want).max()


@pytest.mark.parametrize("maker,fname", [("tiny_mixed", "golden_mixed.npz"), ("tiny_formats", "golden_formats_model.npz")])
def test_mixed_type_layers_match_the_reference(po, seeds, maker, fname):
    """Layers whose q/k/v share a type (the reference fuses them behind its 8-lane norm) beside layers where they do
    not, Q4_K and Q6_K in every projection role (synth.tiny_mixed), and layers in the dispatcher's other formats
    (Q8_0, Q5_K, Q5_0: synth.tiny_formats): oracle bit-identical to the compiled reference's forward_decode_cpu."""
    import os
    from prometorch_amd.testing import synth
    g = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", fname))
    cfg, layers, head = getattr(synth, maker)(seeds["tiny"])
    om = po.OracleModel(cfg, layers, head, 64, kv_fp16=False)
    for i in range(cfg["n_layers"]):
        om.set_kv(i, *synth.make_kv_prefill(seeds["tiny"], i, cfg, 19))
    for st in range(12):
        assert om.step(synth.MIXED_FEED[st]) == int(g["tokens"][st]), st
        assert np.array_equal(bits(om.logits), bits(g["logits"][st])), st


def test_q4k_fp32_activation_variant_vs_reference_scalar_kernel(po, seeds):
    """golden_q4k_f32act.npz: the compiled reference's q4k_gemv_scalar (fp32 activations, no Q8 rounding); the oracle's
    restatement is bit-identical, and equals the float64 product of the dequantised matrix to fp32 rounding."""
    import os
    from conftest import GOLDEN_DIR
    g = np.load(os.path.join(GOLDEN_DIR, "golden_q4k_f32act.npz"), allow_pickle=False)
    for name, N, K in (("a", 96, 2560), ("b", 5, 256)):
        r = synth.rng_for(seeds["blocks"], 31, N)
        W = synth.make_q4k(r, N, K)
        x = synth.make_x(r, K)
        y = po.gemv(12, W, x, "f32")
        assert np.array_equal(bits(y), bits(g["y_" + name])), name
        want = po.dequant(12, W).reshape(N, K).astype(np.float64) @ x.astype(np.float64)
        assert np.abs(y - want).max() / np.sqrt((want ** 2).mean()) < 1e-5


def test_longrope_factors_vs_reference(po, seeds):
    """golden_longrope.npz: the compiled reference's rope_precompute with per-frequency factors and attn_factor, and 12 steps
    of its forward_decode_cpu on a model whose factor set switches from short to long inside the run.  The oracle is
    bit-identical; the C ABI's host table builder too; factors that are all 1 with attn_factor 1 change nothing."""
    import os
    import sys
    from conftest import GOLDEN_DIR
    sys.path.insert(0, GOLDEN_DIR)
    import make_golden as mg
    from prometorch_amd import _lib
    g = np.load(os.path.join(GOLDEN_DIR, "golden_longrope.npz"), allow_pickle=False)
    cfg = mg.longrope_cfg(seeds["tiny"])
    hd = cfg["head_dim"]
    for pos in (0, 1, 21, 22, 2049):
        for which in ("short", "long"):
            c, s = po.rope_tables(pos, hd, cfg["rope_base"], 1.0, cfg["rope_factors_" + which], cfg["rope_attn_factor"])
            assert np.array_equal(bits(c), bits(g["cos_%s_%d" % (which, pos)])), (which, pos)
            assert np.array_equal(bits(s), bits(g["sin_%s_%d" % (which, pos)])), (which, pos)
    # the product's host table: row pos takes the short set while pos + 1 <= orig_ctx
    tab = np.empty((40, hd), np.float32)
    fs, fl = cfg["rope_factors_short"], cfg["rope_factors_long"]
    assert _lib.load().ptm_rope_table_host_factors(tab.ctypes.data, 40, hd, cfg["rope_base"], 1.0, fs.ctypes.data, fl.ctypes.data,
                                                   cfg["rope_orig_ctx"], cfg["rope_attn_factor"]) == 0
    for pos, which in ((0, "short"), (1, "short"), (21, "short"), (22, "long")):
        assert np.array_equal(bits(tab[pos, :hd // 2]), bits(g["cos_%s_%d" % (which, pos)])), pos
        assert np.array_equal(bits(tab[pos, hd // 2:]), bits(g["sin_%s_%d" % (which, pos)])), pos
    plain = np.empty((40, hd), np.float32)
    ones = np.ones(hd // 2, np.float32)
    _lib.load().ptm_rope_table_host_factors(plain.ctypes.data, 40, hd, cfg["rope_base"], 1.0, ones.ctypes.data, ones.ctypes.data, 22, 1.0)
    c0, s0 = po.rope_tables(17, hd, cfg["rope_base"])
    assert np.array_equal(bits(plain[17, :hd // 2]), bits(c0)) and np.array_equal(bits(plain[17, hd // 2:]), bits(s0))
    # the whole step
    layers = [synth.make_layer(seeds["tiny"], i, cfg) for i in range(cfg["n_layers"])]
    head = synth.make_head(seeds["tiny"], cfg)
    om = po.OracleModel(cfg, layers, head, 64, kv_fp16=False)
    for i in range(cfg["n_layers"]):
        om.set_kv(i, *synth.make_kv_prefill(seeds["tiny"], i, cfg, 19))
    tok = 3
    for st in range(12):
        tok = om.step(tok)
        assert tok == int(g["tokens"][st]) and np.array_equal(bits(om.logits), bits(g["logits"][st])), st
    # and the factors matter: the same model without them decodes to different logits
    om2 = po.OracleModel(dict(synth.TINY), layers, head, 64, kv_fp16=False)
    for i in range(cfg["n_layers"]):
        om2.set_kv(i, *synth.make_kv_prefill(seeds["tiny"], i, cfg, 19))
    om2.step(3)
    assert np.abs(om2.logits - g["logits"][0]).max() / g["logits"][0].std() > 1e-2
