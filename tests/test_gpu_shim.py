"""GPU: a decode step issued purely through the reference's launcher names (include/ptm_at_cuda_shim.h, driven by
tests/shim_harness.cpp in the order of GGUFModel::forward_decode), and the operators those names needed beyond the
graph-replayable ones: position from the host, unquantised GEMVs, row rotation, row copies."""
import ctypes as C
import os

import numpy as np
import pytest
import torch

from conftest import ROOT
from prometorch_amd import _lib, ops
from prometorch_amd.testing import synth

pytestmark = pytest.mark.gpu

vp, i64 = C.c_void_p, C.c_int64


class ShimQW(C.Structure):
    _fields_ = [("gpu_data", vp), ("type", C.c_int32), ("rows", C.c_int32), ("cols", C.c_int32), ("row_stride_bytes", i64)]


class ShimLayer(C.Structure):
    _fields_ = [(n, ShimQW) for n in ("q", "k", "v", "o", "gate", "up", "down")] + \
               [(n, vp) for n in ("attn_norm", "ffn_norm", "q_norm", "k_norm", "key_cache", "value_cache")]


class ShimModel(C.Structure):
    _fields_ = [(n, C.c_int32) for n in ("n_layers", "H", "n_heads", "n_kv_heads", "head_dim", "inter", "vocab", "max_seq")] + \
               [("rope_freq_base", C.c_float), ("eps", C.c_float), ("rope_neox", C.c_int32), ("rope_table", vp), ("emb", vp),
                ("layers", C.POINTER(ShimLayer)), ("output_norm", vp), ("lm_head", ShimQW), ("buf_x", vp * 2)] + \
               [(n, vp) for n in ("buf_normed", "buf_q", "buf_k", "buf_v", "buf_attn", "buf_h", "buf_gate", "buf_up", "buf_silu",
                                  "buf_down", "buf_logits", "fd_partial_O", "fd_partial_lse", "fd_partial_max", "d_token_id",
                                  "d_past_len", "d_argmax_idx")]


def harness():
    path = os.path.join(ROOT, "tests", "libshim_harness.so")
    assert os.path.exists(path), "tests/libshim_harness.so is not built (python -c 'import __graft_entry__ as g; g.build()')"
    h = C.CDLL(path)
    h.shim_forward_decode.restype = C.c_int
    h.shim_forward_decode.argtypes = [C.POINTER(ShimModel), C.c_int, i64, vp]
    return h


_KEEP = []


def dev_f32(a):
    """fp32 device copy, kept alive until the test module is torn down (a temporary's memory would be handed to the next
    allocation before the launch that reads it has even been issued)"""
    t = torch.from_numpy(np.ascontiguousarray(a, np.float32)).cuda()
    _KEEP.append(t)
    return t


@pytest.mark.parametrize("graph_style", [1, 0])
@pytest.mark.parametrize("table", [True, False])
def test_decode_step_through_the_reference_launcher_names(dev, po, seeds, graph_style, table):
    """12 tokens of the tiny Q4_K_M model: every launch goes through at::cuda::launch_*; logits against the CPU oracle
    (fp32 KV cache, as the reference's decode keeps it), argmax identical."""
    H = harness()
    cfg = dict(synth.TINY)
    layers = [synth.make_layer(seeds["tiny"], i, cfg) for i in range(cfg["n_layers"])]
    head = synth.make_head(seeds["tiny"], cfg)
    max_seq, past0 = 64, 19
    om = po.OracleModel(cfg, layers, head, max_seq, kv_fp16=False)
    keep = []
    arr = (ShimLayer * cfg["n_layers"])()
    kvd = cfg["n_kv_heads"] * cfg["head_dim"]
    for i, Ld in enumerate(layers):
        for name in ("q", "k", "v", "o", "gate", "up", "down"):
            qt, W = Ld[name]
            t = torch.from_numpy(np.ascontiguousarray(W)).cuda()
            keep.append(t)
            setattr(arr[i], name, ShimQW(t.data_ptr(), qt, W.shape[0], _lib.weight_cols(qt, W.shape[1]), W.shape[1]))
        for name in ("attn_norm", "ffn_norm", "q_norm", "k_norm"):
            t = dev_f32(Ld[name])
            keep.append(t)
            setattr(arr[i], name, t.data_ptr())
        k16, v16 = synth.make_kv_prefill(seeds["tiny"], i, cfg, past0)
        om.set_kv(i, k16, v16)
        kc = torch.zeros(max_seq, kvd, device="cuda")
        vc = torch.zeros(max_seq, kvd, device="cuda")
        kc[:past0] = torch.from_numpy(k16.astype(np.float32))
        vc[:past0] = torch.from_numpy(v16.astype(np.float32))
        keep += [kc, vc]
        arr[i].key_cache, arr[i].value_cache = kc.data_ptr(), vc.data_ptr()
    m = ShimModel()
    m.n_layers, m.H, m.n_heads, m.n_kv_heads = cfg["n_layers"], cfg["hidden"], cfg["n_heads"], cfg["n_kv_heads"]
    m.head_dim, m.inter, m.vocab, m.max_seq = cfg["head_dim"], cfg["inter"], cfg["vocab"], max_seq
    m.rope_freq_base, m.eps, m.rope_neox = cfg["rope_base"], cfg["eps"], 1
    rt = ops.rope_table(max_seq, cfg["head_dim"], cfg["rope_base"]).cuda()
    m.rope_table = rt.data_ptr() if table else None
    emb = dev_f32(po.dequant(14, head["lm_head"]).reshape(cfg["vocab"], cfg["hidden"]))
    lm = torch.from_numpy(np.ascontiguousarray(head["lm_head"])).cuda()
    on = dev_f32(head["out_norm"])
    m.emb, m.layers, m.output_norm = emb.data_ptr(), arr, on.data_ptr()
    m.lm_head = ShimQW(lm.data_ptr(), 14, cfg["vocab"], cfg["hidden"], head["lm_head"].shape[1])
    S = ops._L().ptm_flash_decode_num_splits(max_seq)
    qd = cfg["n_heads"] * cfg["head_dim"]
    bufs = {}
    for name, n in (("x0", cfg["hidden"]), ("x1", cfg["hidden"]), ("buf_normed", cfg["hidden"]), ("buf_q", qd), ("buf_k", kvd),
                    ("buf_v", kvd), ("buf_attn", qd), ("buf_h", cfg["hidden"]), ("buf_gate", cfg["inter"]),
                    ("buf_up", cfg["inter"]), ("buf_silu", cfg["inter"]), ("buf_down", cfg["hidden"]),
                    ("buf_logits", cfg["vocab"]), ("fd_partial_O", S * qd), ("fd_partial_lse", S * cfg["n_heads"]),
                    ("fd_partial_max", S * cfg["n_heads"])):
        bufs[name] = torch.zeros(n, device="cuda")
        if name not in ("x0", "x1"):
            setattr(m, name, bufs[name].data_ptr())
    m.buf_x[0], m.buf_x[1] = bufs["x0"].data_ptr(), bufs["x1"].data_ptr()
    d_tok = torch.zeros(1, dtype=torch.int32, device="cuda")
    d_past = torch.zeros(1, dtype=torch.int64, device="cuda")
    d_arg = torch.zeros(1, dtype=torch.int64, device="cuda")
    m.d_token_id, m.d_past_len, m.d_argmax_idx = d_tok.data_ptr(), d_past.data_ptr(), d_arg.data_ptr()
    tok_o = tok_g = 3
    errs = []
    for st in range(12):
        tok_o = om.step(tok_o)
        d_tok.fill_(tok_g)
        d_past.fill_(past0 + st)
        torch.cuda.synchronize()
        n_calls = H.shim_forward_decode(C.byref(m), graph_style, past0 + st, torch.cuda.current_stream().cuda_stream)
        assert n_calls == 1 + cfg["n_layers"] * 12 + 3, n_calls
        torch.cuda.synchronize()
        tok_g = int(d_arg.item())
        lg = bufs["buf_logits"].cpu().numpy()
        errs.append(float(np.abs(lg - om.logits).max() / om.logits.std()))
        assert tok_g == tok_o, (st, errs[-1])
    # host-libm rotation table: 1e-3 of the logits' spread, a step on a Q8 rounding boundary up to 2e-2 (at most 2);
    # angles computed on the device differ in the last bits, which the Q8 rounding of later products amplifies now and then
    errs = np.asarray(errs)
    assert errs.max() <= 2e-2, errs
    if table:
        assert int((errs > 1e-3).sum()) <= 2, errs
    assert keep and rt is not None and emb is not None and lm is not None and on is not None


def test_flash_decode_pos_equals_device_position_form(dev):
    rng = np.random.default_rng(5)
    n_heads, n_kv, hd, T = 8, 2, 128, 333
    Q = dev_f32(rng.standard_normal(n_heads * hd))
    for kv16 in (0, 1):
        dt = torch.float16 if kv16 else torch.float32
        Kc = torch.from_numpy(rng.standard_normal((T, n_kv * hd)).astype(np.float32)).cuda().to(dt)
        Vc = torch.from_numpy(rng.standard_normal((T, n_kv * hd)).astype(np.float32)).cuda().to(dt)
        S = ops._L().ptm_flash_decode_num_splits(T)
        pO, pL, pM = (torch.zeros(S * n_heads * hd, device="cuda"), torch.zeros(S * n_heads, device="cuda"),
                      torch.zeros(S * n_heads, device="cuda"))
        O1, O2 = torch.zeros(n_heads * hd, device="cuda"), torch.zeros(n_heads * hd, device="cuda")
        past = torch.tensor([T - 1], dtype=torch.int64, device="cuda")
        s = torch.cuda.current_stream().cuda_stream
        L = ops._L()
        _lib.check(L.ptm_flash_decode(Q.data_ptr(), Kc.data_ptr(), Vc.data_ptr(), O1.data_ptr(), pO.data_ptr(), pL.data_ptr(),
                                      pM.data_ptr(), n_heads, n_kv, hd, past.data_ptr(), T, 0.088, kv16, s), "fd")
        _lib.check(L.ptm_flash_decode_pos(Q.data_ptr(), Kc.data_ptr(), Vc.data_ptr(), O2.data_ptr(), pO.data_ptr(),
                                          pL.data_ptr(), pM.data_ptr(), n_heads, n_kv, hd, T, 0.088, kv16, s), "fd_pos")
        torch.cuda.synchronize()
        assert torch.equal(O1, O2) and float(O1.abs().sum()) > 0
        assert L.ptm_flash_decode_pos(Q.data_ptr(), Kc.data_ptr(), Vc.data_ptr(), O2.data_ptr(), pO.data_ptr(), pL.data_ptr(),
                                      pM.data_ptr(), n_heads, n_kv, hd, 0, 0.088, kv16, s) == -6


def test_qknorm_rope_kvwrite_pos_rotates_at_position_and_writes_at_row(dev, po):
    """Rotation position and cache row differ (the reference's non-graph launcher takes both)."""
    rng = np.random.default_rng(6)
    n_heads, n_kv, hd, max_seq, pos, row = 4, 2, 128, 40, 31, 7
    q, k, v = (rng.standard_normal(n_heads * hd).astype(np.float32), rng.standard_normal(n_kv * hd).astype(np.float32),
               rng.standard_normal(n_kv * hd).astype(np.float32))
    qw, kw = 1 + 0.1 * rng.standard_normal(hd).astype(np.float32), 1 + 0.1 * rng.standard_normal(hd).astype(np.float32)
    qn = np.concatenate([po.rmsnorm(q[h * hd:(h + 1) * hd], qw, 1e-6) for h in range(n_heads)])
    kn = np.concatenate([po.rmsnorm(k[h * hd:(h + 1) * hd], kw, 1e-6) for h in range(n_kv)])
    c, s = po.rope_tables(pos, hd, 1e6)
    table = ops.rope_table(max_seq, hd, 1e6).cuda()
    L = ops._L()
    for neox in (1, 0):
        want_q, want_k = (po.rope_neox if neox else po.rope_norm)(qn, kn, c, s, n_heads, n_kv, hd)
        Q, K, V = dev_f32(q), dev_f32(k), dev_f32(v)
        Kc, Vc = torch.zeros(max_seq, n_kv * hd, device="cuda"), torch.zeros(max_seq, n_kv * hd, device="cuda")
        _lib.check(L.ptm_qknorm_rope_kvwrite_pos(Q.data_ptr(), K.data_ptr(), V.data_ptr(), dev_f32(qw).data_ptr(),
                                                 dev_f32(kw).data_ptr(), Kc.data_ptr(), Vc.data_ptr(), n_heads, n_kv, hd, pos,
                                                 row, max_seq, 1e6, table.data_ptr(), 1e-6, 0, neox, 0,
                                                 torch.cuda.current_stream().cuda_stream), "kvwrite_pos")
        torch.cuda.synchronize()
        assert np.abs(Q.cpu().numpy() - want_q).max() < 3e-6 and np.abs(K.cpu().numpy() - want_k).max() < 3e-6
        assert torch.equal(Kc[row], K) and np.array_equal(Vc[row].cpu().numpy(), v)
        assert float(Kc.abs().sum() - Kc[row].abs().sum()) == 0.0   # no other row touched
    assert L.ptm_qknorm_rope_kvwrite_pos(16, 16, 16, None, None, 16, 16, 4, 2, 128, 3, 40, 40, 1e6, None, 1e-6, 0, 1, 0,
                                         None) == -6


def test_plain_operators_against_numpy(dev, po):
    rng = np.random.default_rng(7)
    L = ops._L()
    s = torch.cuda.current_stream().cuda_stream
    K, N = 640, 77
    W = rng.standard_normal((N, K)).astype(np.float32)
    x = rng.standard_normal(K).astype(np.float32)
    want = W.astype(np.float64) @ x.astype(np.float64)
    y = torch.zeros(N, device="cuda")
    _lib.check(L.ptm_f32_gemv(dev_f32(W).data_ptr(), dev_f32(x).data_ptr(), y.data_ptr(), K, N, 0, s), "f32 gemv")
    torch.cuda.synchronize()
    assert np.abs(y.cpu().numpy() - want).max() < 2e-4
    _lib.check(L.ptm_f32_gemv(dev_f32(W.T.copy()).data_ptr(), dev_f32(x).data_ptr(), y.data_ptr(), K, N, 1, s), "f32 gemv kn")
    torch.cuda.synchronize()
    assert np.abs(y.cpu().numpy() - want).max() < 2e-4
    Wh = W.astype(np.float16)
    want_h = Wh.astype(np.float64) @ x.astype(np.float64)
    want_hx = Wh.astype(np.float64) @ x.astype(np.float16).astype(np.float64)
    Whd = torch.from_numpy(Wh).cuda()
    WhTd = torch.from_numpy(np.ascontiguousarray(Wh.T)).cuda()
    for k_major, round_x, w, t in ((0, 0, want_h, Whd), (0, 1, want_hx, Whd), (1, 0, want_h, WhTd), (1, 1, want_hx, WhTd)):
        _lib.check(L.ptm_f16_gemv(t.data_ptr(), dev_f32(x).data_ptr(), y.data_ptr(), K, N, k_major, round_x, s), "f16 gemv")
        torch.cuda.synchronize()
        assert np.abs(y.cpu().numpy() - w).max() < 2e-4, (k_major, round_x)
    # the [K][N] fp16 order is what ptm_dequant_q4k_to_fp16 writes: the pair equals the Q4_K dequantised product
    Wq = synth.make_weight(synth.rng_for(9), 12, 64, 512)
    xq = rng.standard_normal(512).astype(np.float32)
    Wd = torch.from_numpy(Wq).cuda()
    f16 = torch.zeros(512 * 64, dtype=torch.float16, device="cuda")
    ops.launch_dequant_q4k_to_fp16(Wd, f16, 512, 64, Wq.shape[1])
    yq = torch.zeros(64, device="cuda")
    _lib.check(L.ptm_f16_gemv(f16.data_ptr(), dev_f32(xq).data_ptr(), yq.data_ptr(), 512, 64, 1, 0, s), "f16 gemv of dequant")
    torch.cuda.synchronize()
    deq = po.dequant(12, Wq).reshape(64, 512)
    want_q = deq.astype(np.float16).astype(np.float64) @ xq.astype(np.float64)
    assert np.abs(yq.cpu().numpy() - want_q).max() < 1e-3 * np.abs(want_q).max()
    # out-of-place scale, row copy, row concatenation
    a, b = rng.standard_normal((5, 48)).astype(np.float32), rng.standard_normal((3, 48)).astype(np.float32)
    out = torch.zeros(8, 48, device="cuda")
    _lib.check(L.ptm_concat_rows(dev_f32(a).data_ptr(), dev_f32(b).data_ptr(), out.data_ptr(), 5, 3, 48, s), "concat")
    cache = torch.zeros(16, 48, device="cuda")
    _lib.check(L.ptm_kv_cache_write(dev_f32(b).data_ptr(), cache.data_ptr(), 3, 48, 9, s), "kv write")
    sc = torch.zeros(5 * 48, device="cuda")
    _lib.check(L.ptm_mul_scalar(dev_f32(a).data_ptr(), 1.5, sc.data_ptr(), 5 * 48, s), "mul_scalar")
    torch.cuda.synchronize()
    assert np.array_equal(out.cpu().numpy(), np.concatenate([a, b]))
    assert np.array_equal(cache[9:12].cpu().numpy(), b) and float(cache[:9].abs().sum() + cache[12:].abs().sum()) == 0.0
    assert np.array_equal(sc.cpu().numpy(), (a * np.float32(1.5)).ravel())
    # rotation of prompt rows: row r at position 11 + r, both pairings, table and device angles
    n_heads, hd, rows = 3, 64, 4
    data = rng.standard_normal((rows, n_heads * hd)).astype(np.float32)
    table = ops.rope_table(32, hd, 1e4).cuda()
    for neox in (0, 1):
        want = np.empty_like(data)
        for r in range(rows):
            c, sn = po.rope_tables(11 + r, hd, 1e4)
            fn = po.rope_neox if neox else po.rope_norm
            want[r], _ = fn(data[r], data[r][:hd].copy(), c, sn, n_heads, 1, hd)
        for tab, tol in ((table.data_ptr(), 1e-6), (None, 2e-5)):
            d = dev_f32(data)
            _lib.check(L.ptm_rope(d.data_ptr(), rows, n_heads, hd, 11, 1e4, tab, 32, neox, s), "rope")
            torch.cuda.synchronize()
            assert np.abs(d.cpu().numpy() - want).max() < tol, (neox, tab is None)
    assert L.ptm_rope(16, 4, 3, 64, 30, 1e4, 16, 32, 0, None) == -6   # rows run past the table
