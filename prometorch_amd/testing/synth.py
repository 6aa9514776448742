"""Seeded synthetic GGUF k-quant data for the benchmark configurations.

Everything is generated with numpy's PCG64 stream from an explicit seed, so the same
call yields the same bytes wherever it runs.  Block layouts follow the GGUF super-block
formats (reference: torch/io/gguf_dequant.h:158,160,289-297,301-319,392-408).
"""
from __future__ import annotations

import numpy as np

Q4_K, Q6_K = 12, 14
BLOCK_BYTES = {Q4_K: 144, Q6_K: 210}


def rng_for(seed: int, *stream: int) -> np.random.Generator:
    """Independent generator for (seed, stream ids...)."""
    return np.random.Generator(np.random.PCG64(np.random.SeedSequence([seed, *stream])))


def row_stride(qtype: int, cols: int) -> int:
    assert cols % 256 == 0
    return cols // 256 * BLOCK_BYTES[qtype]


def pack_scales_k4(sc: np.ndarray, mn: np.ndarray) -> np.ndarray:
    """Pack 8 six-bit scales and 8 six-bit mins ([..., 8] uint8 each) into [..., 12] bytes,
    the inverse of get_scale_min_k4 (reference: gguf_dequant.h:289-297)."""
    sc = sc.astype(np.uint8)
    mn = mn.astype(np.uint8)
    out = np.empty(sc.shape[:-1] + (12,), dtype=np.uint8)
    out[..., 0:4] = (sc[..., 0:4] & 63) | ((sc[..., 4:8] >> 4) << 6)
    out[..., 4:8] = (mn[..., 0:4] & 63) | ((mn[..., 4:8] >> 4) << 6)
    out[..., 8:12] = (sc[..., 4:8] & 0x0F) | ((mn[..., 4:8] & 0x0F) << 4)
    return out


def make_q4k(rng: np.random.Generator, rows: int, cols: int, d_scale: float = 0.01) -> np.ndarray:
    """[rows, cols/256*144] uint8 of Q4_K super-blocks: d, dmin = fp16(|N(0,1)|*d_scale),
    6-bit scales/mins uniform 0..63, 4-bit quants uniform 0..15."""
    nb = rows * (cols // 256)
    blk = np.empty((nb, 144), dtype=np.uint8)
    dd = (np.abs(rng.standard_normal((nb, 2), dtype=np.float32)) * np.float32(d_scale)).astype(np.float16)
    blk[:, 0:4] = dd.view(np.uint8).reshape(nb, 4)
    sm = rng.integers(0, 64, size=(nb, 16), dtype=np.uint8)
    blk[:, 4:16] = pack_scales_k4(sm[:, :8], sm[:, 8:])
    blk[:, 16:144] = rng.integers(0, 256, size=(nb, 128), dtype=np.uint8)
    return blk.reshape(rows, cols // 256 * 144)


def make_q6k(rng: np.random.Generator, rows: int, cols: int, d_scale: float = 0.005) -> np.ndarray:
    """[rows, cols/256*210] uint8 of Q6_K super-blocks: ql/qh uniform bytes (quants 0..63),
    16 int8 scales uniform -32..31, d = fp16(|N(0,1)|*d_scale)."""
    nb = rows * (cols // 256)
    blk = np.empty((nb, 210), dtype=np.uint8)
    blk[:, 0:192] = rng.integers(0, 256, size=(nb, 192), dtype=np.uint8)
    blk[:, 192:208] = rng.integers(-32, 32, size=(nb, 16), dtype=np.int8).view(np.uint8)
    d = (np.abs(rng.standard_normal((nb, 1), dtype=np.float32)) * np.float32(d_scale)).astype(np.float16)
    blk[:, 208:210] = d.view(np.uint8).reshape(nb, 2)
    return blk.reshape(rows, cols // 256 * 210)


def make_q5k(rng: np.random.Generator, rows: int, cols: int, d_scale: float = 0.01) -> np.ndarray:
    """[rows, cols/256*176] uint8 of Q5_K super-blocks: d, dmin, 6-bit scales/mins as Q4_K, 32 bytes of fifth bits,
    128 bytes of nibbles, all uniform."""
    nb = rows * (cols // 256)
    blk = np.empty((nb, 176), dtype=np.uint8)
    dd = (np.abs(rng.standard_normal((nb, 2), dtype=np.float32)) * np.float32(d_scale)).astype(np.float16)
    blk[:, 0:4] = dd.view(np.uint8).reshape(nb, 4)
    sm = rng.integers(0, 64, size=(nb, 16), dtype=np.uint8)
    blk[:, 4:16] = pack_scales_k4(sm[:, :8], sm[:, 8:])
    blk[:, 16:176] = rng.integers(0, 256, size=(nb, 160), dtype=np.uint8)
    return blk.reshape(rows, cols // 256 * 176)


def make_q8_0(rng: np.random.Generator, rows: int, cols: int, d_scale: float = 0.002) -> np.ndarray:
    """[rows, cols/32*34] uint8 of Q8_0 blocks: d = fp16(|N(0,1)|*d_scale), 32 int8 quants uniform -127..127."""
    nb = rows * (cols // 32)
    blk = np.empty((nb, 34), dtype=np.uint8)
    d = (np.abs(rng.standard_normal((nb, 1), dtype=np.float32)) * np.float32(d_scale)).astype(np.float16)
    blk[:, 0:2] = d.view(np.uint8).reshape(nb, 2)
    blk[:, 2:34] = rng.integers(-127, 128, size=(nb, 32), dtype=np.int8).view(np.uint8)
    return blk.reshape(rows, cols // 32 * 34)


def make_q5_0(rng: np.random.Generator, rows: int, cols: int, d_scale: float = 0.01) -> np.ndarray:
    """[rows, cols/32*22] uint8 of Q5_0 blocks: d = fp16(|N(0,1)|*d_scale), 32 fifth bits, 16 bytes of nibbles."""
    nb = rows * (cols // 32)
    blk = np.empty((nb, 22), dtype=np.uint8)
    d = (np.abs(rng.standard_normal((nb, 1), dtype=np.float32)) * np.float32(d_scale)).astype(np.float16)
    blk[:, 0:2] = d.view(np.uint8).reshape(nb, 2)
    blk[:, 2:22] = rng.integers(0, 256, size=(nb, 20), dtype=np.uint8)
    return blk.reshape(rows, cols // 32 * 22)


Q5_0, Q8_0, Q5_K = 6, 8, 13


def make_weight(rng, qtype: int, rows: int, cols: int) -> np.ndarray:
    return {Q4_K: make_q4k, Q6_K: make_q6k, Q5_K: make_q5k, Q8_0: make_q8_0, Q5_0: make_q5_0}[qtype](rng, rows, cols)


def make_x(rng: np.random.Generator, n: int) -> np.ndarray:
    return rng.standard_normal(n, dtype=np.float32)


# --------------------------------------------------------------------------------------
# closed-form numpy dequantisers (independent of the C oracle; used to pin it)
# --------------------------------------------------------------------------------------
def unpack_scales_k4(q12: np.ndarray):
    """[..., 12] bytes -> (sc[..., 8], mn[..., 8]) per get_scale_min_k4."""
    q = q12.astype(np.uint8)
    sc = np.empty(q.shape[:-1] + (8,), dtype=np.uint8)
    mn = np.empty_like(sc)
    sc[..., 0:4] = q[..., 0:4] & 63
    mn[..., 0:4] = q[..., 4:8] & 63
    sc[..., 4:8] = (q[..., 8:12] & 0x0F) | ((q[..., 0:4] >> 6) << 4)
    mn[..., 4:8] = (q[..., 8:12] >> 4) | ((q[..., 4:8] >> 6) << 4)
    return sc, mn


def dequant_q4k_np(raw: np.ndarray) -> np.ndarray:
    blk = raw.reshape(-1, 144)
    d = blk[:, 0:2].copy().view(np.float16).astype(np.float32)   # [nb,1]
    dmin = blk[:, 2:4].copy().view(np.float16).astype(np.float32)
    sc, mn = unpack_scales_k4(blk[:, 4:16])
    qs = blk[:, 16:144].reshape(-1, 4, 32)
    q = np.stack([qs & 0x0F, qs >> 4], axis=2).reshape(-1, 8, 32).astype(np.float32)  # sub-block order
    ds = (d * sc.astype(np.float32))[:, :, None]
    ms = (dmin * mn.astype(np.float32))[:, :, None]
    return (ds * q - ms).astype(np.float32).reshape(-1)


def dequant_q6k_np(raw: np.ndarray) -> np.ndarray:
    blk = raw.reshape(-1, 210)
    nb = blk.shape[0]
    ql = blk[:, 0:128].reshape(nb, 2, 2, 32)      # [half][which32][l]
    qh = blk[:, 128:192].reshape(nb, 2, 32)
    sc = blk[:, 192:208].copy().view(np.int8).astype(np.float32).reshape(nb, 2, 4, 2)  # [half][grp][l/16]
    d = blk[:, 208:210].copy().view(np.float16).astype(np.float32).reshape(nb, 1, 1, 1)
    out = np.empty((nb, 2, 4, 32), dtype=np.float32)
    for grp in range(4):
        lo = ql[:, :, grp & 1, :]
        nib = (lo >> 4) if (grp & 2) else (lo & 0x0F)
        q = (nib | (((qh >> (2 * grp)) & 3) << 4)).astype(np.int32) - 32
        s = np.repeat(sc[:, :, grp, :], 16, axis=-1)          # [nb,2,32]
        out[:, :, grp, :] = (d[:, :, 0, :] * s) * q.astype(np.float32)
    return out.reshape(-1)


# --------------------------------------------------------------------------------------
# model-shaped bundles
# --------------------------------------------------------------------------------------
QWEN3_4B = dict(vocab=151936, hidden=2560, n_layers=36, n_heads=32, n_kv_heads=8, head_dim=128,
                inter=9728, rope_base=1.0e6, eps=1.0e-6)
TINY = dict(vocab=1024, hidden=256, n_layers=2, n_heads=4, n_kv_heads=2, head_dim=64,
            inter=512, rope_base=1.0e6, eps=1.0e-6)

# (name, quant type, rows-key, cols-key) for the Q4_K_M mix: v and down in Q6_K
LAYER_MATS = (("q", Q4_K), ("k", Q4_K), ("v", Q6_K), ("o", Q4_K), ("gate", Q4_K), ("up", Q4_K), ("down", Q6_K))


def layer_shapes(cfg: dict) -> dict:
    H, qd, kvd, I = cfg["hidden"], cfg["n_heads"] * cfg["head_dim"], cfg["n_kv_heads"] * cfg["head_dim"], cfg["inter"]
    return {"q": (qd, H), "k": (kvd, H), "v": (kvd, H), "o": (H, qd), "gate": (I, H), "up": (I, H), "down": (H, I)}


# Scale of the RMSNorm weights (gamma = scale * (1 + 0.1*N(0,1))).  The super-block
# distributions of the benchmark configurations give weights of magnitude ~1.5 with a fan-in
# of 2560..9728, i.e. a gain of ~100 per projection; with unit gammas every layer overwrites
# the residual stream and the random network is chaotic (last-bit differences grow to O(1)
# within a few tokens).  These gammas keep each branch's output at the scale of the residual,
# as in a trained model, so that greedy decoding is a well-conditioned function of the inputs.
NORM_SCALE = {"attn": 0.1, "ffn": 1.0e-3, "qk": 1.0, "out": 1.0}


def make_layer(seed: int, layer: int, cfg: dict, norm_scale: dict | None = None, mats=None) -> dict:
    """One decoder layer's seven weight matrices plus its four norm vectors
    (gamma = scale * (1 + 0.1*N(0,1)), scale per NORM_SCALE).  mats: (name, quant type) pairs, LAYER_MATS by default."""
    ns = dict(NORM_SCALE if norm_scale is None else norm_scale)
    shp = layer_shapes(cfg)
    out = {}
    for i, (name, qt) in enumerate(LAYER_MATS if mats is None else mats):
        out[name] = (qt, make_weight(rng_for(seed, 1, layer, i), qt, *shp[name]))
    g = rng_for(seed, 2, layer)
    for name, n, sc in (("attn_norm", cfg["hidden"], ns["attn"]), ("ffn_norm", cfg["hidden"], ns["ffn"]),
                        ("q_norm", cfg["head_dim"], ns["qk"]), ("k_norm", cfg["head_dim"], ns["qk"])):
        gam = np.float32(1.0) + np.float32(0.1) * g.standard_normal(n, dtype=np.float32)
        out[name] = (np.float32(sc) * gam).astype(np.float32)
    return out


def center_q4k(W: np.ndarray) -> np.ndarray:
    """The Q4_K super-blocks of W with their mins set equal to their scales and dmin = fp16(7.5 d): a block then holds
    d * scale * (q - 7.5), values symmetric about zero.  (make_q4k's independent scales and mins give every weight a large
    positive mean, d * 31.5 * 7.5 - dmin * 31.5; a network of such matrices is close to rank one - whatever token is fed, its
    logits point along one of two directions.)"""
    rows = W.shape[0]
    blk = W.reshape(-1, 144).copy()
    sc, _ = unpack_scales_k4(blk[:, 4:16])
    blk[:, 4:16] = pack_scales_k4(sc, sc)
    d = blk[:, 0:2].copy().view(np.float16).astype(np.float32)
    blk[:, 2:4] = (np.float32(7.5) * d).astype(np.float16).view(np.uint8).reshape(-1, 2)
    return blk.reshape(rows, -1)


def make_layer_centered(seed: int, layer: int, cfg: dict, norm_scale: dict | None = None) -> dict:
    """make_layer with every Q4_K matrix centred (center_q4k): the same seeds, scales and quants."""
    L = make_layer(seed, layer, cfg, norm_scale)
    for name, _ in LAYER_MATS:
        qt, W = L[name]
        if qt == Q4_K:
            L[name] = (qt, center_q4k(W))
    return L


def make_head(seed: int, cfg: dict) -> dict:
    """Tied Q6_K token-embedding / lm_head table and the output norm."""
    g = rng_for(seed, 3)
    return {
        "lm_head": make_q6k(g, cfg["vocab"], cfg["hidden"]),
        "out_norm": (np.float32(1.0) + np.float32(0.1) * g.standard_normal(cfg["hidden"], dtype=np.float32)).astype(np.float32),
    }


def make_kv_prefill(seed: int, layer: int, cfg: dict, n_pos: int):
    """fp16 K/V cache contents for positions [0, n_pos): N(0,1) rounded to fp16."""
    g = rng_for(seed, 4, layer)
    kvd = cfg["n_kv_heads"] * cfg["head_dim"]
    k = g.standard_normal((n_pos, kvd), dtype=np.float32).astype(np.float16)
    v = g.standard_normal((n_pos, kvd), dtype=np.float32).astype(np.float16)
    return k, v


# Type mixes a Q4_K_M file really holds besides LAYER_MATS (about half of its layers keep attn_v and ffn_down in
# Q4_K), and one it does not, to reach the remaining branches of the step (a Q6_K q beside Q4_K k and v, Q6_K o and gate)
MIX_ALL_Q4K = tuple((n, Q4_K) for n, _ in LAYER_MATS)
MIX_ODD = (("q", Q6_K), ("k", Q4_K), ("v", Q4_K), ("o", Q6_K), ("gate", Q6_K), ("up", Q4_K), ("down", Q6_K))


# The dispatcher's other formats in every projection role: a Q8_0 layer, a Q5_K layer, and a layer mixing all five types
MIX_Q8_0 = tuple((n, Q8_0) for n, _ in LAYER_MATS)
MIX_Q5_K = tuple((n, Q5_K) for n, _ in LAYER_MATS)
MIX_FIVE = (("q", Q5_0), ("k", Q8_0), ("v", Q5_K), ("o", Q4_K), ("gate", Q5_K), ("up", Q8_0), ("down", Q5_0))


def tiny_formats(seed: int):
    """The TINY shapes with three layers in the GEMV dispatcher's other formats: MIX_Q8_0, MIX_Q5_K, MIX_FIVE."""
    cfg = dict(TINY)
    cfg["n_layers"] = 3
    layers = [make_layer(seed, i, cfg, mats=m) for i, m in enumerate((MIX_Q8_0, MIX_Q5_K, MIX_FIVE))]
    return cfg, layers, make_head(seed, cfg)


MIXED_FEED = tuple((131 * i + 3) % 1024 for i in range(32))  # tokens fed to tiny_mixed step by step


def tiny_mixed(seed: int):
    """The TINY shapes with three layers of different type mixes: LAYER_MATS, MIX_ALL_Q4K, MIX_ODD."""
    cfg = dict(TINY)
    cfg["n_layers"] = 3
    layers = [make_layer(seed, i, cfg, mats=m) for i, m in enumerate((LAYER_MATS, MIX_ALL_Q4K, MIX_ODD))]
    return cfg, layers, make_head(seed, cfg)


LLAMA3_8B = dict(vocab=128256, hidden=4096, n_layers=32, n_heads=32, n_kv_heads=8, head_dim=128,
                 inter=14336, rope_base=5.0e5, eps=1.0e-5, rope_interleaved=True)


def llama3_8b_like(seed: int, n_layers: int = 2, vocab: int = 32000):
    """Llama-3-8B layer shapes (no QK-norm, interleaved rotation), a few layers and a reduced vocabulary so that the
    CPU oracle can step it; attention-input norm gains reduced as in tiny_llama."""
    cfg = dict(LLAMA3_8B)
    cfg["n_layers"], cfg["vocab"] = n_layers, vocab
    layers = [make_layer(seed, i, cfg) for i in range(n_layers)]
    for L in layers:
        L["q_norm"] = None
        L["k_norm"] = None
        L["attn_norm"] = (np.float32(0.1) * L["attn_norm"]).astype(np.float32)
    return cfg, layers, make_head(seed, cfg)


QWEN25_7B = dict(vocab=152064, hidden=3584, n_layers=28, n_heads=28, n_kv_heads=4, head_dim=128, inter=18944,
                 rope_base=1.0e6, eps=1.0e-6)


def qwen25_7b_like(seed: int, n_layers: int = 2, vocab: int = 32000):
    """Qwen2.5-7B layer shapes (7 query heads per kv head, q / k / v biases, no QK-norm; 14 and 74 super-blocks per row),
    a few layers and a reduced vocabulary so that the CPU oracle can step it; attention-input norm gains reduced as in
    tiny_llama."""
    cfg = dict(QWEN25_7B)
    cfg["n_layers"], cfg["vocab"] = n_layers, vocab
    layers = [make_layer(seed, i, cfg) for i in range(n_layers)]
    qd, kvd = cfg["n_heads"] * cfg["head_dim"], cfg["n_kv_heads"] * cfg["head_dim"]
    for i, L in enumerate(layers):
        L["q_norm"] = None
        L["k_norm"] = None
        L["attn_norm"] = (np.float32(0.1) * L["attn_norm"]).astype(np.float32)
        g = rng_for(seed, 5, i)
        for name, n in (("q_bias", qd), ("k_bias", kvd), ("v_bias", kvd)):
            L[name] = (np.float32(0.5) * g.standard_normal(n, dtype=np.float32)).astype(np.float32)
    return cfg, layers, make_head(seed, cfg)


GEMMA3_4B = dict(vocab=262144, hidden=2560, n_layers=34, n_heads=8, n_kv_heads=4, head_dim=256, inter=10240,
                 rope_base=1.0e6, eps=1.0e-6, scale_embeddings=True, ffn_gelu=True, swa_window=1024, swa_pattern=6,
                 rope_swa_base=1.0e4, rope_scale=8.0)


def gemma3_4b_like(seed: int, n_layers: int = 2, vocab: int = 32000):
    """Gemma-3-4B layer shapes (256-wide heads, post-norms, GELU gate, five local layers of window 1024 per global one),
    optionally with fewer layers and a reduced vocabulary so that the CPU oracle can step it."""
    cfg = dict(GEMMA3_4B)
    cfg["n_layers"], cfg["vocab"] = n_layers, vocab
    layers = [make_layer(seed, i, cfg) for i in range(n_layers)]
    for i, L in enumerate(layers):
        g = rng_for(seed, 6, i)
        for name in ("post_attn_norm", "post_ffn_norm"):
            L[name] = (np.float32(0.5) * (np.float32(1.0) + np.float32(0.1) * g.standard_normal(cfg["hidden"], dtype=np.float32))).astype(np.float32)
    return cfg, layers, make_head(seed, cfg)


def tiny_llama(seed: int):
    """The TINY shapes as a llama-style model: no per-head QK-norm, interleaved rotation pairs.  The attention-input
    norm weights are a tenth of TINY's: with random weights and no QK-norm the Q.K scores would otherwise run to the
    hundreds, softmax would pick one position outright and neither the rotation nor the cache would matter."""
    cfg = dict(TINY)
    cfg["rope_interleaved"] = True
    layers = [make_layer(seed, i, cfg) for i in range(cfg["n_layers"])]
    for L in layers:
        L["q_norm"] = None
        L["k_norm"] = None
        L["attn_norm"] = (np.float32(0.1) * L["attn_norm"]).astype(np.float32)
    return cfg, layers, make_head(seed, cfg)


def tiny_qwen2(seed: int):
    """The TINY shapes as a qwen2-style model: no per-head QK-norm, NeoX rotation pairs, and bias vectors on the q, k and
    v projections (N(0,1) scaled to the size of the projections' outputs, so that dropping one changes the tokens).
    Attention-input norm gains reduced as in tiny_llama."""
    cfg = dict(TINY)
    layers = [make_layer(seed, i, cfg) for i in range(cfg["n_layers"])]
    qd, kvd = cfg["n_heads"] * cfg["head_dim"], cfg["n_kv_heads"] * cfg["head_dim"]
    for i, L in enumerate(layers):
        L["q_norm"] = None
        L["k_norm"] = None
        L["attn_norm"] = (np.float32(0.1) * L["attn_norm"]).astype(np.float32)
        g = rng_for(seed, 5, i)
        for name, n in (("q_bias", qd), ("k_bias", kvd), ("v_bias", kvd)):
            L[name] = (np.float32(0.5) * g.standard_normal(n, dtype=np.float32)).astype(np.float32)
    return cfg, layers, make_head(seed, cfg)


def tiny_gemma(seed: int, n_layers: int = 4, head_dim: int = 64):
    """The TINY shapes as a gemma3-style model: embedding rows times sqrt(hidden), per-head QK-norm, NeoX rotation,
    tanh-GELU gate, RMSNorm on each branch's output before the residual add, and alternating attention: layers li with
    (li + 1) % 3 != 0 see only the last 8 positions and rotate with base 1e4, the others see everything and rotate with
    base 1e6 and positions divided by 8.  Four layers: local, local, global, local.  head_dim = 256 gives gemma3's head
    width.  The embedding scale of 16 is undone in
    the first norm gains' scale so that activations stay where the other tiny models have them."""
    cfg = dict(TINY, n_layers=n_layers, scale_embeddings=True, ffn_gelu=True, swa_window=8, swa_pattern=3, rope_swa_base=1.0e4,
               rope_scale=8.0)
    if head_dim != cfg["head_dim"]:  # gemma3's heads are 256 wide: two query heads on one kv head, q_dim 512
        cfg.update(head_dim=head_dim, n_heads=2, n_kv_heads=1)
    layers = [make_layer(seed, i, cfg) for i in range(n_layers)]
    for i, L in enumerate(layers):
        g = rng_for(seed, 6, i)
        for name in ("post_attn_norm", "post_ffn_norm"):
            L[name] = (np.float32(0.5) * (np.float32(1.0) + np.float32(0.1) * g.standard_normal(cfg["hidden"], dtype=np.float32))).astype(np.float32)
    return cfg, layers, make_head(seed, cfg)


def random_model(seed):
    """A small decoder with every architectural switch drawn at random: head width, query heads per kv head, QK-norm or
    none, rotation pairing, position scaling, q / k / v biases, the gemma features each on its own, the type of every
    matrix from the tuned pair."""
    r = rng_for(97, seed)
    hd = int(r.choice([64, 128, 256]))
    G = int(r.integers(1, 9))
    nkv = int(r.integers(1, 3))
    nh = G * nkv
    while (nh * hd) % 256:   # q_dim must hold whole super-blocks
        nkv += 1
        nh = G * nkv
    cfg = dict(vocab=512, hidden=int(r.choice([256, 512, 768])), n_layers=int(r.integers(2, 5)), n_heads=nh, n_kv_heads=nkv,
               head_dim=hd, inter=256 * int(r.integers(1, 5)), rope_base=float(r.choice([1.0e4, 1.0e6])), eps=1.0e-6)
    if r.random() < 0.5:
        cfg["rope_interleaved"] = True
    if r.random() < 0.4:
        cfg["rope_scale"] = float(r.choice([2.0, 8.0]))
    if r.random() < 0.5:
        cfg["scale_embeddings"] = True
    if r.random() < 0.5:
        cfg["ffn_gelu"] = True
    if r.random() < 0.5:
        cfg.update(swa_window=int(r.integers(1, 40)), swa_pattern=int(r.integers(1, 4)), rope_swa_base=1.0e4)
    qk_norm, bias = r.random() < 0.5, r.random() < 0.5
    post = [r.random() < 0.5, r.random() < 0.5]
    layers = []
    for i in range(cfg["n_layers"]):
        mats = tuple((n, int(r.choice([Q4_K, Q6_K]))) for n in ("q", "k", "v", "o", "gate", "up", "down"))
        L = make_layer(1000 + seed, i, cfg, mats=mats)
        L["attn_norm"] = (np.float32(0.1) * L["attn_norm"]).astype(np.float32)
        if not qk_norm:
            L["q_norm"] = L["k_norm"] = None
        g = rng_for(98, seed, i)
        if bias:
            for name, n in (("q_bias", nh * hd), ("k_bias", nkv * hd), ("v_bias", nkv * hd)):
                L[name] = (np.float32(0.5) * g.standard_normal(n, dtype=np.float32)).astype(np.float32)
        for on, name in zip(post, ("post_attn_norm", "post_ffn_norm")):
            if on:
                L[name] = (np.float32(0.5) * (1 + np.float32(0.1) * g.standard_normal(cfg["hidden"], dtype=np.float32))).astype(np.float32)
        layers.append(L)
    return cfg, layers, make_head(1000 + seed, cfg)


# ---- sampling cases: (vocab, logit kind, temperature, top_k, top_p), in the order the golden run draws them ----
SAMPLING_CASES = (
    [(1000, "normal", 0.8, 40, 0.9), (1000, "normal", 1.0, 0, 1.0), (1000, "normal", 0.7, 1, 1.0),
     (1000, "ties", 1.0, 40, 0.9), (1000, "ties", 1.5, 100, 0.5), (1000, "normal", 0.0, 40, 0.9),
     (1000, "normal", 0.8, 0, 0.9), (1000, "peaked", 2.0, 5, 0.3), (1000, "normal", 1.0, 40, 1.0),
     (1000, "normal", 0.8, 1000, 0.95), (1000, "negative", 0.8, 40, 0.9), (37, "normal", 0.8, 40, 0.9)]
    + [(151936, "normal", 0.8, 40, 0.9)] * 6 + [(151936, "ties", 0.8, 40, 0.9), (151936, "peaked", 1.2, 64, 0.8),
                                                  (151936, "normal", 0.6, 0, 0.9), (151936, "normal", 1.0, 1024, 1.0)]
    + [(1000, "normal", 0.9, 50, 0.85)] * 24
)


def sampling_logits(case_index: int) -> np.ndarray:
    """Logits of sampling case i.  normal: 3 N(0,1); ties: the same rounded to 0.25 (equal values around the
    k-th largest); peaked: one token far ahead; negative: all below zero."""
    vocab, kind = SAMPLING_CASES[case_index][:2]
    g = rng_for(4242, case_index)
    x = np.float32(3.0) * g.standard_normal(vocab, dtype=np.float32)
    if kind == "ties":
        x = (np.round(x * 4) / 4).astype(np.float32)
    elif kind == "peaked":
        x[int(g.integers(0, vocab))] += np.float32(12.0)
    elif kind == "negative":
        x = (-np.abs(x) - np.float32(1.0)).astype(np.float32)
    return x


# ---- synthetic tokenizers: a small trained BPE per kind, and the texts the golden run encodes ----
_CORPUS = (
    "The quick brown fox jumps over the lazy dog. It's 2024, isn't it? They're here; we'll see what you've done.\n"
    "I'd say she's right: 3.14159 is close to pi, and 1000000 is a million!  Tabs\tand  double  spaces   matter.\n"
    "def encode(text):\n    return [ord(c) for c in text]  # comment\n\nfor i in range(10): print(i, i * i)\n"
    "Привет, мир! Как дела? Это тест токенизатора: числа 12345 и знаки препинания...\n"
    "你好，世界！这是一个分词器的测试。日本語のテキストも少し。\n"
    "Emoji \U0001F600 and symbols éèüß € 100 — done. <tag> not special </tag>\n"
    "the the the and and of of to to in in that that is is was was he he for for it it with with as as his his\n"
)

_SPECIALS = ["<|endoftext|>", "<|im_start|>", "<|im_end|>", "<think>", "</think>"]


def _byte_char(b: int) -> str:
    """GPT-2 bytes_to_unicode."""
    if (33 <= b <= 126) or (161 <= b <= 172) or (174 <= b <= 255):
        return chr(b)
    if b <= 32:
        return chr(0x100 + b)
    if 127 <= b <= 160:
        return chr(0x121 + b - 127)
    return chr(0x143)


def _train_bpe(words: dict, n_merges: int) -> list:
    """words: tuple of symbols -> count.  Classic BPE training: merge the most frequent adjacent pair, repeatedly."""
    merges = []
    words = dict(words)
    for _ in range(n_merges):
        pairs = {}
        for w, c in words.items():
            for a, b in zip(w, w[1:]):
                pairs[(a, b)] = pairs.get((a, b), 0) + c
        if not pairs:
            break
        (a, b), _ = max(pairs.items(), key=lambda kv: (kv[1], kv[0]))
        merges.append((a, b))
        nw = {}
        for w, c in words.items():
            out, i = [], 0
            while i < len(w):
                if i + 1 < len(w) and w[i] == a and w[i + 1] == b:
                    out.append(a + b)
                    i += 2
                else:
                    out.append(w[i])
                    i += 1
            nw[tuple(out)] = nw.get(tuple(out), 0) + c
        words = nw
    return merges


def make_tokenizer(kind: str, n_merges: int = 300, vocab_size: int | None = None) -> dict:
    """kind 'gpt2': byte-level BPE (256 byte symbols, merges over space-prefixed words, ChatML-style specials);
    'llama': word-marker BPE over UTF-8 characters with <0xNN> byte tokens; 'greedy': the llama vocabulary without
    merges (longest-match mode).  Returns the tokenizer.ggml.* metadata."""
    import re
    if kind == "gpt2":
        words = {}
        for m in re.finditer(r" ?[^\W\d_]+| ?\d+| ?[^\s\w]+|\s+", _CORPUS):
            w = tuple(_byte_char(b) for b in m.group(0).encode("utf-8"))
            words[w] = words.get(w, 0) + 1
        merges = _train_bpe(words, n_merges)
        vocab = [_byte_char(b) for b in range(256)] + [a + b for a, b in merges] + _SPECIALS
        if vocab_size:  # padded to a model's vocabulary with reserved specials
            vocab += ["<|reserved_%d|>" % i for i in range(vocab_size - len(vocab))]
        eos = vocab.index("<|endoftext|>")
        return {"tokenizer.ggml.model": "gpt2", "tokenizer.ggml.tokens": vocab,
                "tokenizer.ggml.merges": [a + " " + b for a, b in merges], "tokenizer.ggml.bos_token_id": eos,
                "tokenizer.ggml.eos_token_id": eos, "tokenizer.ggml.padding_token_id": eos,
                "tokenizer.ggml.add_bos_token": False}
    words = {}
    for w in _CORPUS.replace("\n", " ").replace("\t", " ").split(" "):
        if w:
            t = tuple("▁" + w)
            words[t] = words.get(t, 0) + 1
    merges = _train_bpe(words, n_merges)
    chars = sorted({c for w in words for c in w} - {"д"})          # one Cyrillic letter left out: byte fallback
    vocab = ["<unk>", "<s>", "</s>"] + ["<0x%02X>" % b for b in range(256)] + chars + [a + b for a, b in merges] + ["\n"]
    md = {"tokenizer.ggml.model": "llama", "tokenizer.ggml.tokens": vocab,
          "tokenizer.ggml.scores": [0.0] * len(vocab), "tokenizer.ggml.bos_token_id": 1,
          "tokenizer.ggml.eos_token_id": 2, "tokenizer.ggml.unknown_token_id": 0, "tokenizer.ggml.add_bos_token": True}
    if kind == "llama":
        md["tokenizer.ggml.merges"] = [a + " " + b for a, b in merges]
    return md


def tokenizer_texts(kind: str) -> list:
    """Byte strings the golden run encodes.  For 'gpt2' none has a UTF-8 continuation byte that does not follow a
    letter byte: the reference's splitter does not terminate on those."""
    fixed = [
        "", " ", "  ", "a", "Hello, world!", "hello world", " leading and trailing ", "two  spaces   three", "tabs\tand\nnewlines\r\n\n",
        "It's what they're saying: I'd, we'll, you've, he's, I'm, don't 'quoted' 'tis", "'s", "'", "x'", "x'r", "x're",
        "1234567890 3.14 2024-05-06 1,000", "snake_case CamelCase kebab-case path/to/file.py", "!!! ... ??? --- (()) [[ ]] {{}}",
        "Привет, мир! Как дела?", "Сегодня 5 мая, погода хорошая.", "你好，世界！", "日本語のテキスト", "emoji \U0001F600\U0001F680 end",
        "café naïve über straße €5", "<|im_start|>user\nHi<|im_end|>\n<|im_start|>assistant\n",
        "<think>hmm</think>ok<|endoftext|>", "<|im_start|><|im_end|><|im_start|>", "a<b>c <0x41> <tag> <|unknown|> <>", "<s>x</s><unk>",
        "the the the and of to in that is was", "def f(x):\n    return x * 2  # twice\n", "line1\n\nline3\n   indented\n\ttabbed",
        "trailing spaces   ", "\n", "\n\n\n", " \n \n", "a\nb", "MiXeD 123abc456 abc123", "▁marker▁inside", "ĠG-dot Ċ",
        "д д дд один два", "x" * 70, "ab" * 40 + " " + "the" * 30,
    ]
    out = [t.encode("utf-8") for t in fixed]
    out += [b"\xffabc", b"a\x80\x81b", b"ok \xe4\xbd", b"\xc3(", b"\xc0\xc1 odd", b"abc\xf0\x9f\x98"]   # malformed UTF-8 that is safe for both splitters
    g = rng_for(5151, 1 if kind == "gpt2" else 2)
    alphabet = list("abcdefghijklmnopqrstuvwxyzTHE    \n\t.,!?'0123456789") + ["the", " and", "'s", "'re", "д", "ы", "你", "\U0001F600", "<|im_end|>", "<s>", "é"]
    for _ in range(40):
        n = int(g.integers(1, 60))
        out.append("".join(alphabet[int(i)] for i in g.integers(0, len(alphabet), n)).encode("utf-8"))
    if kind != "gpt2":
        out += [bytes(g.integers(0, 256, int(g.integers(1, 40)), dtype=np.uint8)) for _ in range(20)]        # arbitrary bytes
    return out
