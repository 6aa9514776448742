"""GPU parity: the HIP kernels, called through the C ABI, against the CPU oracle and the golden
vectors of the compiled reference, on identical seeded inputs.

Bars: dequantised weights and Q8 activation blocks bit-exact; GEMV outputs within 1e-3 of the
oracle relative to rms(y) (fp32 accumulation, same Q8 activation handling); argmax / greedy token
ids identical."""
import numpy as np
import pytest
import torch

from conftest import bits, sha, sha_of
from prometorch_amd import ops
from prometorch_amd.testing import synth

pytestmark = pytest.mark.gpu

GEMV_TOL = 1e-3  # max |y_gpu - y_cpu| / rms(y_cpu), the bar the path is specified to


def cu(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def rel_err(y, ref):
    ref = ref.astype(np.float64)
    return float(np.abs(y.astype(np.float64) - ref).max() / max(np.sqrt((ref ** 2).mean()), 1e-30))


def gpu_gemv(qt, W, x, accumulate=False, y0=None):
    N, stride = W.shape
    K = x.size
    Wd, xd = cu(W), cu(x)
    y = cu(y0) if y0 is not None else torch.full((N,), 123.0, device="cuda")
    ops.quant_gemv(qt, Wd, xd, y, K, N, stride, accumulate=accumulate)
    torch.cuda.synchronize()
    return y.cpu().numpy()


# ---------------------------------------------------------------------------------------------
# dequantisation, fp16, Q8
# ---------------------------------------------------------------------------------------------
@pytest.mark.parametrize("qt,key", [(12, "q4k"), (14, "q6k")])
def test_dequant_bit_exact_golden(dev, golden, qt, key):
    raw = golden[key + "_blocks"]
    n = raw.shape[0] * 256
    out = torch.empty(n, device="cuda")
    (ops.dequant_q4k if qt == 12 else ops.dequant_q6k)(cu(raw), out, n)
    torch.cuda.synchronize()
    assert np.array_equal(bits(out.cpu().numpy()), bits(golden[key + "_deq"]))


def test_fp16_conversion_all_65536_values(dev, po):
    # one Q4_K block per fp16 pattern h: d = h, scale 1, quant 1, min 0  =>  weight == fp16_to_fp32(h)
    blk = np.zeros((65536, 144), np.uint8)
    blk[:, 0:2] = np.arange(65536, dtype=np.uint16).view(np.uint8).reshape(-1, 2)
    blk[:, 4:16] = synth.pack_scales_k4(np.ones((65536, 8), np.uint8), np.zeros((65536, 8), np.uint8))
    blk[:, 16:144] = 0x11
    out = torch.empty(65536 * 256, device="cuda")
    ops.dequant_q4k(cu(blk), out, 65536 * 256)
    torch.cuda.synchronize()
    got = out.cpu().numpy().reshape(65536, 256)
    want = np.arange(65536, dtype=np.uint16).view(np.float16).astype(np.float32)
    # the block computes d*1*1 - dmin*0, i.e. d + (-0.0): identical to d except that it maps -0 to... -0 - 0 = -0
    fin = np.isfinite(want)
    assert np.array_equal(bits(got[fin, 0]), bits(want[fin])), "fp16 -> fp32 (incl. subnormals) is not exact"
    assert np.all(got[fin] == got[fin, :1])
    # and the oracle agrees on every finite pattern
    assert np.array_equal(bits(po.dequant(12, blk[fin][:, :144])[::256]), bits(want[fin]))


def test_dequant_full_cfg1_matrix_bit_exact(dev, po, seeds):
    r = synth.rng_for(seeds["cfg1"])
    W = synth.make_q4k(r, 9728, 2560)
    n = 9728 * 2560
    out = torch.empty(n, device="cuda")
    ops.dequant_q4k(cu(W), out, n)
    torch.cuda.synchronize()
    assert sha(out.cpu().numpy()) == sha(po.dequant(12, W))
    r6 = synth.rng_for(seeds["cfg3"], 77)
    W6 = synth.make_q6k(r6, 2560, 9728)
    out6 = torch.empty(2560 * 9728, device="cuda")
    ops.dequant_q6k(cu(W6), out6, 2560 * 9728)
    torch.cuda.synchronize()
    assert sha(out6.cpu().numpy()) == sha(po.dequant(14, W6))


def test_dequant_q4k_to_fp16_column_major(dev, po):
    W = synth.make_q4k(synth.rng_for(21), 48, 512)
    out = torch.empty(512, 48, dtype=torch.float16, device="cuda")
    ops.launch_dequant_q4k_to_fp16(cu(W), out, 512, 48, W.shape[1])
    torch.cuda.synchronize()
    want = po.dequant(12, W).reshape(48, 512).T.astype(np.float16)
    assert np.array_equal(out.cpu().numpy().view(np.uint16), want.view(np.uint16))


def q8_unpack(buf, K):
    raw = buf.cpu().numpy()
    qs = raw[:K].view(np.int8)
    f = raw[K:K + K // 4].view(np.float32)
    return f[:K // 32], f[K // 32:], qs


def test_quantize_q8_bit_exact(dev, po, golden):
    x = golden["q8_x"]
    buf = torch.zeros(ops.q8_bytes(2560), dtype=torch.uint8, device="cuda")
    ops.launch_quantize_q8(cu(x), buf, 2560)
    torch.cuda.synchronize()
    d, s, q = q8_unpack(buf, 2560)
    assert np.array_equal(q, golden["q8_qs"])
    assert np.array_equal(bits(d), bits(golden["q8_d"]))
    assert np.array_equal(bits(s), bits(golden["q8_sum"]))
    # a second, larger vector with a wide dynamic range, against the oracle
    rng = synth.rng_for(22)
    x2 = (synth.make_x(rng, 9728) * np.exp(rng.standard_normal(9728) * 3)).astype(np.float32)
    buf2 = torch.zeros(ops.q8_bytes(9728), dtype=torch.uint8, device="cuda")
    ops.launch_quantize_q8(cu(x2), buf2, 9728)
    torch.cuda.synchronize()
    d2, s2, q2 = q8_unpack(buf2, 9728)
    do, so, qo = po.quantize_x_q8(x2)
    assert np.array_equal(q2, qo) and np.array_equal(bits(d2), bits(do)) and np.array_equal(bits(s2), bits(so))


# ---------------------------------------------------------------------------------------------
# GEMV
# ---------------------------------------------------------------------------------------------
def test_q4k_gemv_cfg1(dev, po, golden, seeds):
    r = synth.rng_for(seeds["cfg1"])
    W = synth.make_q4k(r, 9728, 2560)
    x = synth.make_x(r, 2560)
    y = gpu_gemv(12, W, x)
    ref = po.gemv(12, W, x)
    assert sha(ref) == sha_of(golden, "cfg1_sha")  # the comparator is the reference's own output
    e = rel_err(y, ref)
    print("cfg1 q4k gemv rel err", e)
    assert e <= GEMV_TOL
    big = np.abs(ref) > 1e-2 * np.sqrt((ref.astype(np.float64) ** 2).mean())
    assert np.all(np.abs(y[big] - ref[big]) <= GEMV_TOL * np.abs(ref[big]))
    # homogeneity: scaling x by a power of two scales every Q8 block scale exactly, so y doubles bit for bit
    y2 = gpu_gemv(12, W, (x * 2).astype(np.float32))
    assert np.array_equal(bits(y2), bits(y * 2))
    # accumulate form: y0 + W.x
    y0 = synth.make_x(r, 9728)
    ya = gpu_gemv(12, W, x, accumulate=True, y0=y0)
    assert np.array_equal(bits(ya), bits(y0 + y))


def test_q4k_gemv_prequantized_matches_inkernel(dev, seeds):
    r = synth.rng_for(seeds["cfg1"], 1)
    W = synth.make_q4k(r, 4096, 2560)
    x = synth.make_x(r, 2560)
    Wd, xd = cu(W), cu(x)
    y1 = torch.empty(4096, device="cuda")
    y2 = torch.empty(4096, device="cuda")
    q8 = torch.empty(ops.q8_bytes(2560), dtype=torch.uint8, device="cuda")
    ops.launch_q4km_persistent_gemv(Wd, xd, y1, 2560, 4096, W.shape[1])
    ops.launch_quantize_q8(xd, q8, 2560)
    ops.launch_q4km_q8_gemv(Wd, q8, y2, 2560, 4096, W.shape[1])
    torch.cuda.synchronize()
    assert torch.equal(y1, y2)


def test_q4k_gemv_tall_forms_agree(dev, po, seeds):
    """The kernel for very tall Q4_K matrices (block loads rolling across a workgroup's row tiles) in its three forms - fp32
    x, Q8 blocks handed in, accumulate - against the oracle and against each other."""
    r = synth.rng_for(seeds["cfg1"], 7)
    N, K = 40007, 2560
    W = synth.make_q4k(r, N, K)
    x = synth.make_x(r, K)
    ref = po.gemv(12, W, x)
    y = gpu_gemv(12, W, x)
    assert rel_err(y, ref) <= GEMV_TOL
    Wd, xd = cu(W), cu(x)
    y2 = torch.empty(N, device="cuda")
    q8 = torch.empty(ops.q8_bytes(K), dtype=torch.uint8, device="cuda")
    ops.launch_quantize_q8(xd, q8, K)
    ops.launch_q4km_q8_gemv(Wd, q8, y2, K, N, W.shape[1])
    torch.cuda.synchronize()
    assert np.array_equal(bits(y2.cpu().numpy()), bits(y))
    y0 = synth.make_x(r, N)
    ya = gpu_gemv(12, W, x, accumulate=True, y0=y0)
    assert np.array_equal(bits(ya), bits(y0 + y))


@pytest.mark.parametrize("N,K", [(2560, 9728), (3584, 18944), (4099, 14336), (5120, 25600), (2001, 11008), (2560, 4096)])
def test_q4k_gemv_long_rows_equal_the_general_kernel(dev, N, K):
    """One matrix of few long rows with fp32 x takes the one-row-per-wave kernel (x quantised once per workgroup); with Q8
    blocks handed in, or as the first of three matrices of one launch, the same rows take the general kernel.  Same
    block-to-lane assignment and reduction order, so the same bits - with 8 to 16 waves, one to three half blocks of x per
    thread, one and two workgroups per CU."""
    r = synth.rng_for(37, N, K)
    W = synth.make_q4k(r, N, K)
    x = synth.make_x(r, K)
    y = gpu_gemv(12, W, x)
    Wd, xd = cu(W), cu(x)
    y2 = torch.empty(N, device="cuda")
    q8 = torch.empty(ops.q8_bytes(K), dtype=torch.uint8, device="cuda")
    ops.launch_quantize_q8(xd, q8, K)
    ops.launch_q4km_q8_gemv(Wd, q8, y2, K, N, W.shape[1])
    yq, yk, yv = torch.empty(N, device="cuda"), torch.empty(1, device="cuda"), torch.empty(1, device="cuda")
    ops.launch_q4km_fused_qkv_gemv(Wd, Wd[:1], Wd[:1], xd, yq, yk, yv, K, N, 1, 1, W.shape[1])
    torch.cuda.synchronize()
    assert np.array_equal(bits(y2.cpu().numpy()), bits(y))
    assert np.array_equal(bits(yq.cpu().numpy()), bits(y))
    y0 = synth.make_x(r, N)
    y3 = cu(y0)
    ops.launch_q4km_q8_gemv(Wd, q8, y3, K, N, W.shape[1], accumulate=True)
    torch.cuda.synchronize()
    assert np.array_equal(bits(y3.cpu().numpy()), bits(y0 + y))


def test_q4k_gemv_long_rows_accumulate(dev, po, seeds):
    """The few-long-rows Q4_K kernel (2560 x 9728) in its accumulating form: y0 + W.x, bit for bit the sum of y0 and the plain
    form's result."""
    r = synth.rng_for(seeds["cfg1"], 9)
    W = synth.make_q4k(r, 2560, 9728)
    x = synth.make_x(r, 9728)
    y = gpu_gemv(12, W, x)
    assert rel_err(y, po.gemv(12, W, x)) <= GEMV_TOL
    y0 = synth.make_x(r, 2560)
    ya = gpu_gemv(12, W, x, accumulate=True, y0=y0)
    assert np.array_equal(bits(ya), bits(y0 + y))


@pytest.mark.parametrize("qt,N,K", [(12, 33, 512), (12, 1, 256), (12, 77, 2560), (14, 7, 256), (14, 45, 1024),
                                    (12, 2560, 4096), (12, 2560, 9728), (14, 2560, 9728), (14, 1024, 2560),
                                    (12, 31, 32768), (14, 5, 16384),
                                    # very tall Q4_K matrices: a workgroup walks several row tiles and the block loads roll
                                    # across them (two lane groups per row / one; 5, 2 and 3 blocks per group; ragged last tile)
                                    (12, 40007, 2560), (12, 50001, 512), (12, 45013, 1280), (12, 41000, 768),
                                    # few long Q4_K rows (a Q4_K down projection): one row per wave, x quantised once per
                                    # workgroup; ragged last workgroup, 2 / 5 blocks per lane group, 8 to 12 waves
                                    (12, 2001, 9728), (12, 3000, 10240), (12, 2560, 6144),
                                    # the same with 13 to 16 waves, with two and three half blocks of x per thread, and with
                                    # two workgroups per CU (17 to 32 rows per CU)
                                    (12, 3584, 18944), (12, 4096, 4096), (12, 4099, 14336), (12, 5120, 25600), (12, 6007, 8192)])
def test_gemv_shapes_vs_oracle(dev, po, qt, N, K):
    r = synth.rng_for(31, qt, N, K)
    W = synth.make_weight(r, qt, N, K)
    x = synth.make_x(r, K)
    y = gpu_gemv(qt, W, x)
    ref = po.gemv(qt, W, x)
    e = rel_err(y, ref)
    print(qt, N, K, "rel err", e)
    assert e <= GEMV_TOL


def test_gemv_ragged_vs_reference_golden(dev, golden, seeds):
    rr = synth.rng_for(seeds["ragged"])
    for i, (qt, N, K) in enumerate([(12, 33, 512), (12, 1, 256), (12, 77, 2560), (14, 7, 256), (14, 45, 1024)]):
        W = synth.make_weight(rr, qt, N, K)
        x = synth.make_x(rr, K)
        assert rel_err(gpu_gemv(qt, W, x), golden[f"ragged{i}_y"]) <= GEMV_TOL


def test_gemv_extreme_inputs(dev, po):
    r = synth.rng_for(32)
    W = synth.make_q4k(r, 64, 1024)
    for x in (np.zeros(1024, np.float32),                                   # all-zero activations: d = 0 blocks
              np.where(np.arange(1024) % 32 == 0, 1e30, 0).astype(np.float32),  # one huge value per block
              (synth.make_x(r, 1024) * 1e-30).astype(np.float32)):          # tiny but normal
        y, ref = gpu_gemv(12, W, x), po.gemv(12, W, x)
        if np.any(ref != 0):
            assert rel_err(y, ref) <= GEMV_TOL
        else:
            assert np.all(y == 0)
    W6 = synth.make_q6k(r, 64, 1024)
    x = np.zeros(1024, np.float32)
    assert np.all(gpu_gemv(14, W6, x) == 0)


def test_q6k_accumulate_and_row_stride_padding(dev, po):
    r = synth.rng_for(33)
    N, K = 300, 2560
    W = synth.make_q6k(r, N, K)
    x = synth.make_x(r, K)
    y0 = synth.make_x(r, N)
    ref = po.gemv(14, W, x)
    ya = gpu_gemv(14, W, x, accumulate=True, y0=y0)
    assert rel_err(ya - y0, ref) <= GEMV_TOL
    # rows padded to a larger stride (a row-slice view of a wider tensor)
    pad = np.zeros((N, W.shape[1] + 420), np.uint8)
    pad[:, :W.shape[1]] = W
    pad[:, W.shape[1]:] = 0xAB
    assert np.array_equal(gpu_gemv(14, pad, x), gpu_gemv(14, W, x))
    W4 = synth.make_q4k(r, N, K)
    pad4 = np.full((N, W4.shape[1] + 288), 0xCD, np.uint8)
    pad4[:, :W4.shape[1]] = W4
    assert np.array_equal(gpu_gemv(12, pad4, x), gpu_gemv(12, W4, x))


def test_cfg2_lm_head_gemv_argmax_full_size(dev, po, golden, seeds):
    r = synth.rng_for(seeds["cfg2"])
    W = synth.make_q6k(r, 151936, 2560)
    x = synth.make_x(r, 2560)
    Wd, xd = cu(W), cu(x)
    logits = torch.empty(151936, device="cuda")
    idx = torch.zeros(1, dtype=torch.int64, device="cuda")
    ws = torch.empty(ops.argmax_workspace_bytes(151936), dtype=torch.uint8, device="cuda")
    ops.q6k_gemv_argmax(Wd, xd, logits, 2560, 151936, W.shape[1], idx, ws)
    torch.cuda.synchronize()
    y = logits.cpu().numpy()
    assert int(idx.item()) == int(golden["cfg2_argmax"][0])
    assert int(idx.item()) == int(np.argmax(y))
    top = golden["cfg2_top8_idx"]
    assert np.abs(y[top] - golden["cfg2_top8_val"]).max() <= GEMV_TOL * np.abs(golden["cfg2_top8_val"]).max()
    assert list(np.argsort(-y, kind="stable")[:8]) == list(top)
    ref = po.gemv(14, W, x)
    assert sha(ref) == sha_of(golden, "cfg2_sha")
    e = rel_err(y, ref)
    print("cfg2 q6k lm_head rel err", e)
    assert e <= GEMV_TOL
    # argmax-only form (no logits written) and the standalone argmax agree
    idx2 = torch.zeros(1, dtype=torch.int64, device="cuda")
    ops.q6k_gemv_argmax(Wd, xd, None, 2560, 151936, W.shape[1], idx2, ws)
    idx3 = torch.zeros(1, dtype=torch.int64, device="cuda")
    ops.launch_argmax(logits, idx3, 151936)
    torch.cuda.synchronize()
    assert idx2.item() == idx.item() == idx3.item()


def test_cfg3_layer_gemvs(dev, po, golden, seeds):
    L = synth.make_layer(seeds["cfg3"], 0, synth.QWEN3_4B)
    for i, (name, qt) in enumerate(synth.LAYER_MATS):
        _, W = L[name]
        K = W.shape[1] // (144 if qt == 12 else 210) * 256
        x = synth.make_x(synth.rng_for(seeds["cfg3"], 5, i), K)
        y = gpu_gemv(qt, W, x)
        ref = po.gemv(qt, W, x)
        assert sha(ref) == sha_of(golden, f"cfg3_{name}_sha")
        e = rel_err(y, ref)
        print("cfg3", name, "rel err", e)
        assert e <= GEMV_TOL


def test_fused_gemv_variants(dev, po, golden, seeds):
    L = synth.make_layer(seeds["cfg3"], 0, synth.QWEN3_4B)
    H = 2560
    x = (synth.make_x(synth.rng_for(seeds["cfg3"], 6), H) * 3.0).astype(np.float32)
    gam = L["ffn_norm"]
    xn = po.rmsnorm(x, gam, 1e-6)
    Wg, Wu, Wq, Wk = (cu(L[n][1]) for n in ("gate", "up", "q", "k"))
    stride = L["gate"][1].shape[1]
    xd, gd = cu(x), cu(gam)
    yg = torch.empty(9728, device="cuda")
    yu = torch.empty(9728, device="cuda")
    ops.launch_q4km_fused_rmsnorm_gate_up_gemv(xd, gd, Wg, Wu, yg, yu, H, 9728, 9728, stride, 1e-6, False)
    torch.cuda.synchronize()
    ref_g, ref_u = po.gemv(12, L["gate"][1], xn), po.gemv(12, L["up"][1], xn)
    # the reference's own CPU fusion (cpu_fused_rmsnorm_gate_up_gemv) produced these samples
    assert np.array_equal(bits(ref_g[::152][:64]), bits(golden["cfg3_fused_gate_y64"]))
    assert rel_err(yg.cpu().numpy(), ref_g) <= GEMV_TOL and rel_err(yu.cpu().numpy(), ref_u) <= GEMV_TOL
    # + SiLU*up in the same launch
    act = torch.empty(9728, device="cuda")
    ops.fused_rmsnorm_gate_up_silu(xd, gd, Wg, Wu, act, H, 9728, stride, 1e-6, False)
    torch.cuda.synchronize()
    assert rel_err(act.cpu().numpy(), po.silu_mul(ref_g, ref_u)) <= GEMV_TOL
    # unfused two-matrix and three-matrix launches on a plain x
    xnd = cu(xn)
    y1 = torch.empty(9728, device="cuda")
    y2 = torch.empty(9728, device="cuda")
    ops.launch_q4km_fused_gate_up_gemv(Wg, Wu, xnd, y1, y2, H, 9728, 9728, stride)
    oq = torch.empty(4096, device="cuda")
    ok = torch.empty(1024, device="cuda")
    ov = torch.empty(1024, device="cuda")
    ops.launch_q4km_fused_qkv_gemv(Wq, Wk, Wk, xnd, oq, ok, ov, H, 4096, 1024, 1024, stride)
    oq2 = torch.empty(4096, device="cuda")
    ok2 = torch.empty(1024, device="cuda")
    ov2 = torch.empty(1024, device="cuda")
    ops.launch_q4km_fused_rmsnorm_qkv_gemv(xd, gd, Wq, Wk, Wk, oq2, ok2, ov2, H, 4096, 1024, 1024, stride, 1e-6, False)
    y3 = torch.empty(4096, device="cuda")
    ops.launch_q4km_fused_rmsnorm_gemv(xd, gd, Wq, y3, H, 4096, stride, 1e-6, False)
    torch.cuda.synchronize()
    assert rel_err(y1.cpu().numpy(), ref_g) <= GEMV_TOL and rel_err(y2.cpu().numpy(), ref_u) <= GEMV_TOL
    ref_q, ref_k = po.gemv(12, L["q"][1], xn), po.gemv(12, L["k"][1], xn)
    for got, ref in ((oq, ref_q), (ok, ref_k), (ov, ref_k), (oq2, ref_q), (ok2, ref_k), (ov2, ref_k), (y3, ref_q)):
        assert rel_err(got.cpu().numpy(), ref) <= GEMV_TOL


@pytest.mark.parametrize("N,K", [(14336, 4096), (11003, 2560), (30001, 1024)])
def test_fused_gate_up_silu_tall_shapes_vs_oracle(dev, po, N, K):
    """Gate / up pairs with more row tiles than a launch has workgroups (Llama-3-8B: 2 x 14336 x 4096): a workgroup walks
    several tiles and the block loads roll across them; 4, 5 and 2 blocks per lane group, a ragged last tile."""
    r = synth.rng_for(57, N, K)
    Wg, Wu = synth.make_q4k(r, N, K), synth.make_q4k(r, N, K)
    x = (synth.make_x(r, K) * 2.0).astype(np.float32)
    gam = (1.0 + 0.1 * r.standard_normal(K)).astype(np.float32) * np.float32(0.05)
    xn = po.rmsnorm(x, gam, 1e-6)
    ref = po.silu_mul(po.gemv(12, Wg, xn), po.gemv(12, Wu, xn))
    act = torch.empty(N, device="cuda")
    ops.fused_rmsnorm_gate_up_silu(cu(x), cu(gam), cu(Wg), cu(Wu), act, K, N, Wg.shape[1], 1e-6, False)
    torch.cuda.synchronize()
    got = act.cpu().numpy()
    assert np.all(np.isfinite(got))
    # The launch normalises and quantises x itself: where its RMS scale differs from the oracle's in the last bit, an
    # activation on a Q8 rounding boundary lands on the neighbouring int8 level and every output moves by up to ~1e-2 of the
    # outputs' rms (the decode tests bound the same effect).  A wrong block, row or pairing would be an error of order 1
    # everywhere: the bar is the usual one on the median element and the rounding-step one on the worst.
    rms = np.sqrt((ref.astype(np.float64) ** 2).mean())
    err = np.abs(got.astype(np.float64) - ref) / rms
    print("gate/up", N, K, "median err %.2e max %.2e" % (np.median(err), err.max()))
    assert np.median(err) <= GEMV_TOL and err.max() <= 2e-2


# ---------------------------------------------------------------------------------------------
# glue
# ---------------------------------------------------------------------------------------------
def test_rms_norm_and_q8_output(dev, po, golden):
    x, g = golden["rms_x"], golden["rms_g"]
    out = torch.empty(2560, device="cuda")
    q8 = torch.zeros(ops.q8_bytes(2560), dtype=torch.uint8, device="cuda")
    ops.launch_rms_norm(cu(x), cu(g), out, 1, 2560, 1e-6, False, q8_out=q8)
    torch.cuda.synchronize()
    o = out.cpu().numpy()
    assert np.abs(o - golden["rms_out"]).max() <= 1e-6 * np.abs(golden["rms_out"]).max()
    d, s, q = q8_unpack(q8, 2560)
    do, so, qo = po.quantize_x_q8(o)  # Q8 of what the kernel itself produced: must be bit-exact
    assert np.array_equal(q, qo) and np.array_equal(bits(d), bits(do)) and np.array_equal(bits(s), bits(so))
    rows = np.stack([synth.make_x(synth.rng_for(41, i), 1000) for i in range(5)])
    gam = (1 + 0.1 * synth.make_x(synth.rng_for(41, 9), 1000)).astype(np.float32)
    out2 = torch.empty(5, 1000, device="cuda")
    ops.launch_rms_norm(cu(rows), cu(gam), out2, 5, 1000, 1e-5, True)
    torch.cuda.synchronize()
    r64 = rows.astype(np.float64)
    want = r64 / np.sqrt((r64 ** 2).mean(1, keepdims=True) + 1e-5) * (1 + gam)
    assert np.abs(out2.cpu().numpy() - want).max() < 1e-5
    ph = cu(rows[:, :768].copy())
    ops.launch_per_head_rms_norm(ph, cu(gam[:128]), 5, 6, 128, 1e-6, False)
    torch.cuda.synchronize()
    h64 = rows[:, :768].reshape(5, 6, 128).astype(np.float64)
    wanth = h64 / np.sqrt((h64 ** 2).mean(2, keepdims=True) + 1e-6) * gam[:128]
    assert np.abs(ph.cpu().numpy().reshape(5, 6, 128) - wanth).max() < 1e-5


@pytest.mark.parametrize("kv_fp16", [True, False])
@pytest.mark.parametrize("use_table", [True, False])
def test_qknorm_rope_kvwrite(dev, po, kv_fp16, use_table):
    nh, nkv, hd, max_seq, pos = 32, 8, 128, 2304, 2048
    r = synth.rng_for(42)
    q, k, v = synth.make_x(r, nh * hd) * 5, synth.make_x(r, nkv * hd) * 5, synth.make_x(r, nkv * hd)
    qw = (1 + 0.1 * synth.make_x(r, hd)).astype(np.float32)
    kw = (1 + 0.1 * synth.make_x(r, hd)).astype(np.float32)
    # oracle: per-head RMSNorm, NeoX RoPE with host tables
    qn = np.concatenate([po.rmsnorm(q[h * hd:(h + 1) * hd], qw, 1e-6) for h in range(nh)])
    kn = np.concatenate([po.rmsnorm(k[h * hd:(h + 1) * hd], kw, 1e-6) for h in range(nkv)])
    c, s = po.rope_tables(pos, hd, 1e6)
    qr, kr = po.rope_neox(qn, kn, c, s, nh, nkv, hd)
    dt = torch.float16 if kv_fp16 else torch.float32
    Kc = torch.zeros(max_seq, nkv * hd, dtype=dt, device="cuda")
    Vc = torch.zeros(max_seq, nkv * hd, dtype=dt, device="cuda")
    Q, K, V = cu(q.astype(np.float32)), cu(k.astype(np.float32)), cu(v.astype(np.float32))
    past = torch.tensor([pos], dtype=torch.int64, device="cuda")
    table = ops.rope_table(max_seq, hd, 1e6).cuda() if use_table else None
    ops.launch_fused_qknorm_rope_kvwrite_graph(Q, K, V, cu(qw), cu(kw), Kc, Vc, nh, nkv, hd, past, 1e6, 1e-6, False,
                                               max_seq=max_seq, rope_table=table, neox=True, kv_fp16=kv_fp16)
    torch.cuda.synchronize()
    tol = 2e-6 if use_table else 2e-4  # device sin/cos of theta ~ 2e3 rad differ from libm in the last bits
    assert np.abs(Q.cpu().numpy() - qr).max() <= tol * np.abs(qr).max()
    assert np.abs(K.cpu().numpy() - kr).max() <= tol * np.abs(kr).max()
    krow, vrow = Kc[pos].float().cpu().numpy(), Vc[pos].float().cpu().numpy()
    if kv_fp16:
        assert np.array_equal(vrow, v.astype(np.float32).astype(np.float16).astype(np.float32))
        assert np.array_equal(krow, K.cpu().numpy().astype(np.float16).astype(np.float32))  # RNE of what was computed
    else:
        assert np.array_equal(vrow, v.astype(np.float32)) and np.array_equal(krow, K.cpu().numpy())
    assert float(Kc[:pos].abs().max()) == 0 and float(Kc[pos + 1:].abs().max()) == 0  # only row pos written
    # out-of-range position: nothing is written
    Kc.zero_()
    past.fill_(max_seq)
    ops.launch_fused_qknorm_rope_kvwrite_graph(Q, K, V, cu(qw), cu(kw), Kc, Vc, nh, nkv, hd, past, 1e6, 1e-6, False,
                                               max_seq=max_seq, rope_table=table, neox=True, kv_fp16=kv_fp16)
    torch.cuda.synchronize()
    assert float(Kc.abs().max()) == 0


def test_rope_interleaved_pairs(dev):
    nh, nkv, hd = 4, 2, 64
    r = synth.rng_for(43)
    q, k, v = synth.make_x(r, nh * hd), synth.make_x(r, nkv * hd), synth.make_x(r, nkv * hd)
    Kc = torch.zeros(16, nkv * hd, device="cuda")
    Vc = torch.zeros(16, nkv * hd, device="cuda")
    Q, K = cu(q), cu(k)
    past = torch.tensor([5], dtype=torch.int64, device="cuda")
    ops.launch_fused_qknorm_rope_kvwrite_graph(Q, K, cu(v), None, None, Kc, Vc, nh, nkv, hd, past, 10000.0, 1e-6, False,
                                               max_seq=16, rope_table=None, neox=False, kv_fp16=False)
    torch.cuda.synchronize()
    th = 5.0 * 10000.0 ** (-2 * np.arange(hd // 2) / hd)
    q64 = q.reshape(nh, hd // 2, 2).astype(np.float64)
    want = np.stack([q64[..., 0] * np.cos(th) - q64[..., 1] * np.sin(th),
                     q64[..., 0] * np.sin(th) + q64[..., 1] * np.cos(th)], axis=-1).reshape(-1)
    assert np.abs(Q.cpu().numpy() - want).max() < 1e-5


@pytest.mark.parametrize("kv_fp16", [True, False])
@pytest.mark.parametrize("nh,nkv,hd,T", [(32, 8, 128, 2049), (32, 8, 128, 2176), (4, 2, 64, 20), (8, 8, 128, 1),
                                         (16, 2, 64, 64), (8, 8, 64, 65), (8, 4, 256, 2049), (2, 1, 256, 70), (4, 4, 256, 1), (28, 4, 128, 2049), (6, 2, 64, 100), (5, 1, 128, 65), (6, 2, 256, 90)])
def test_flash_decode_vs_oracle(dev, po, kv_fp16, nh, nkv, hd, T):
    max_seq = max(64, ((T + 127) // 64) * 64)
    r = synth.rng_for(44, nh, hd, T)
    kvd = nkv * hd
    q = synth.make_x(r, nh * hd)
    k16 = r.standard_normal((max_seq, kvd), dtype=np.float32).astype(np.float16)
    v16 = r.standard_normal((max_seq, kvd), dtype=np.float32).astype(np.float16)
    kf, vf = k16.astype(np.float32), v16.astype(np.float32)
    scale = 1.0 / np.sqrt(hd)
    want = np.concatenate([po.attn_head(q[h * hd:(h + 1) * hd], kf, vf, T, kvd, hd, scale, col0=(h // (nh // nkv)) * hd)
                           for h in range(nh)])
    S = ops.flash_decode_num_splits(max_seq)
    pO = torch.empty(S * nh * hd, device="cuda")
    pL = torch.empty(S * nh, device="cuda")
    pM = torch.empty(S * nh, device="cuda")
    O = torch.empty(nh * hd, device="cuda")
    past = torch.tensor([T - 1], dtype=torch.int64, device="cuda")
    Kc, Vc = (cu(k16), cu(v16)) if kv_fp16 else (cu(kf), cu(vf))
    # poison rows past T: they must not be read into the result
    if T < max_seq:
        Kc[T:] = float("nan")
        Vc[T:] = float("nan")
    ops.launch_flash_decode_graph(cu(q), Kc, Vc, O, pO, pL, pM, nh, nkv, hd, past, max_seq, scale, kv_fp16=kv_fp16)
    torch.cuda.synchronize()
    got = O.cpu().numpy()
    assert np.all(np.isfinite(got))
    assert np.abs(got - want).max() <= 2e-5 * max(np.abs(want).max(), 1e-3) + 1e-6


def test_elementwise_embedding_argmax(dev, po):
    r = synth.rng_for(45)
    g = (synth.make_x(r, 9728) * 30).astype(np.float32)
    u = synth.make_x(r, 9728)
    o = torch.empty(9728, device="cuda")
    ops.launch_silu_mul(cu(g), cu(u), o, 9728)
    want = po.silu_mul(g, u)
    torch.cuda.synchronize()
    assert np.abs(o.cpu().numpy() - want).max() <= 1e-6 * np.abs(want).max()
    a, b = synth.make_x(r, 2560), synth.make_x(r, 2560)
    s = torch.empty(2560, device="cuda")
    ops.launch_add(cu(a), cu(b), s, 2560)
    c = torch.empty(2560, device="cuda")
    ops.launch_copy(cu(a), c, 2560)
    torch.cuda.synchronize()
    assert np.array_equal(s.cpu().numpy(), a + b) and np.array_equal(c.cpu().numpy(), a)
    table = r.standard_normal((50, 2560), dtype=np.float32)
    tok = torch.tensor([37], dtype=torch.int32, device="cuda")
    e = torch.empty(2560, device="cuda")
    ops.launch_embedding_lookup(cu(table), e, tok, 2560)
    W6 = synth.make_q6k(r, 50, 2560)
    e6 = torch.empty(2560, device="cuda")
    ops.embedding_lookup_q6k(cu(W6), e6, tok, 2560, W6.shape[1])
    torch.cuda.synchronize()
    assert np.array_equal(e.cpu().numpy(), table[37])
    assert np.array_equal(bits(e6.cpu().numpy()), bits(po.dequant(14, W6[37:38])))
    x = synth.make_x(r, 151936)
    x[[900, 70000, 151935]] = 50.0
    idx = torch.zeros(1, dtype=torch.int64, device="cuda")
    ops.launch_argmax(cu(x), idx, 151936)
    torch.cuda.synchronize()
    assert idx.item() == 900  # strict '>' : the lowest index wins a tie
    src = r.standard_normal((3, 1024), dtype=np.float32)
    cache = torch.zeros(8, 1024, dtype=torch.float16, device="cuda")
    ops.launch_fp16_kv_cache_write(cu(src), cache, 3, 1024, 2)
    torch.cuda.synchronize()
    assert np.array_equal(cache[2:5].cpu().numpy().view(np.uint16), src.astype(np.float16).view(np.uint16))
    assert float(cache[:2].abs().max()) == 0 and float(cache[5:].abs().max()) == 0


@pytest.mark.parametrize("kv_fp16", [True, False])
@pytest.mark.parametrize("nh,nkv,hd,past", [(32, 8, 128, 2048), (32, 8, 128, 2111), (32, 8, 128, 2112), (4, 2, 64, 19),
                                            (8, 8, 128, 0), (16, 2, 64, 63), (8, 1, 64, 64), (8, 8, 64, 130), (4, 2, 64, 29),
                                            (4, 2, 64, 31), (16, 2, 64, 61), (32, 8, 128, 14), (32, 8, 128, 62), (4, 4, 128, 5),
                                            (28, 4, 128, 2100), (40, 8, 128, 300), (12, 2, 128, 70), (24, 8, 64, 19),  # 7, 5, 6, 3 query heads per kv head
                                            (32, 8, 128, 20000),    # past the ~12 k positions where the reference's kernel stops
                                            # caches beyond 4096 positions take the looping kernel: one and several chunks per
                                            # workgroup, a last workgroup with fewer chunks, the new position first / last in its
                                            # chunk, other head shapes
                                            (32, 8, 128, 4090), (8, 2, 128, 4159), (8, 2, 128, 4160), (28, 4, 128, 8191), (4, 2, 64, 8192),
                                            (16, 2, 64, 12345), (40, 8, 128, 6000)])
def test_attn_decode_fused_vs_oracle(dev, po, kv_fp16, nh, nkv, hd, past):
    """QK-norm + RoPE + KV append + attention + merge in one launch, three tokens in a row, against the oracle's pieces in the reference's order."""
    max_seq = ((past + 3 + 63) // 64 + 1) * 64
    r = synth.rng_for(46, nh, hd, past)
    kvd = nkv * hd
    k16 = r.standard_normal((max_seq, kvd), dtype=np.float32).astype(np.float16)
    v16 = r.standard_normal((max_seq, kvd), dtype=np.float32).astype(np.float16)
    kf, vf = k16.astype(np.float32), v16.astype(np.float32)
    qw = (1 + 0.1 * synth.make_x(r, hd)).astype(np.float32)
    kw = (1 + 0.1 * synth.make_x(r, hd)).astype(np.float32)
    dt = torch.float16 if kv_fp16 else torch.float32
    Kc, Vc = cu(kf).to(dt), cu(vf).to(dt)
    Kc[past:] = float("nan")   # rows at and past the new position must not leak into the result
    Vc[past:] = float("nan")
    S = ops.flash_decode_num_splits(max_seq)
    pO = torch.empty(S * nh * hd, device="cuda")
    pL = torch.empty(S * nh, device="cuda")
    pM = torch.empty(S * nh, device="cuda")
    table = ops.rope_table(max_seq, hd, 1e6).cuda()
    O = torch.empty(nh * hd, device="cuda")
    d_past = torch.zeros(1, dtype=torch.int64, device="cuda")
    scale = 1.0 / np.sqrt(hd)
    for step in range(3):
        pos = past + step
        q = (synth.make_x(r, nh * hd) * 3).astype(np.float32)
        k = (synth.make_x(r, kvd) * 3).astype(np.float32)
        v = synth.make_x(r, kvd)
        qn = np.concatenate([po.rmsnorm(q[h * hd:(h + 1) * hd], qw, 1e-6) for h in range(nh)])
        kn = np.concatenate([po.rmsnorm(k[h * hd:(h + 1) * hd], kw, 1e-6) for h in range(nkv)])
        c, s = po.rope_tables(pos, hd, 1e6)
        qr, kr = po.rope_neox(qn, kn, c, s, nh, nkv, hd)
        kf[pos] = kr.astype(np.float16).astype(np.float32) if kv_fp16 else kr
        vf[pos] = v.astype(np.float16).astype(np.float32) if kv_fp16 else v
        want = np.concatenate([po.attn_head(qr[h * hd:(h + 1) * hd], kf, vf, pos + 1, kvd, hd, scale,
                                            col0=(h // (nh // nkv)) * hd) for h in range(nh)])
        d_past.fill_(pos)
        Q, K, V = cu(q), cu(k), cu(v)
        ops.attn_decode_fused(Q, K, V, cu(qw), cu(kw), Kc, Vc, O, pO, pL, pM, table, nh, nkv, hd, d_past,
                              max_seq, scale, 1e-6, kv_fp16=kv_fp16)
        torch.cuda.synchronize()
        got = O.cpu().numpy()
        assert np.all(np.isfinite(got)), (step, pos)
        assert np.abs(got - want).max() <= 3e-5 * max(np.abs(want).max(), 1e-3) + 1e-6, (step, pos)
        assert np.array_equal(Q.cpu().numpy(), q)                    # inputs untouched
        krow = Kc[pos].float().cpu().numpy()
        assert np.abs(krow - kf[pos]).max() <= (2e-3 if kv_fp16 else 2e-6) * np.abs(kf[pos]).max()
        assert np.array_equal(Vc[pos].float().cpu().numpy(), vf[pos])
        kf[pos] = krow                                               # continue from what the cache really holds


@pytest.mark.parametrize("N,K,accumulate", [(2500, 9728, True), (300, 4096, False), (77, 14336, True), (3000, 6912, False),
                                            (4096, 14336, True), (3300, 8192, False), (5119, 13824, False),  # two rows per wave
                                            # rows beyond 14336 values (more than 64 KB of LDS), 13 to 16 waves per workgroup
                                            (3584, 18944, True), (3200, 16384, False), (4001, 20480, False), (5120, 17408, True),
                                            # x in two rounds of loads per thread
                                            (5120, 25600, True), (2100, 27648, False)])
def test_q6k_long_rows_few_rows_vs_oracle(dev, po, N, K, accumulate):
    """Shapes served by the one-row-per-wave kernel (whole x staged once per workgroup): ragged row counts, both
    store modes, and a row stride wider than the row."""
    r = synth.rng_for(34, N, K)
    W = synth.make_q6k(r, N, K)
    x = synth.make_x(r, K)
    ref = po.gemv(14, W, x)
    if accumulate:
        y0 = synth.make_x(r, N)
        y = gpu_gemv(14, W, x, accumulate=True, y0=y0) - y0
        assert rel_err(y, ref) <= 2e-6 * max(1.0, np.abs(y0).max() / np.sqrt((ref ** 2).mean())) + GEMV_TOL * 1e-2
    else:
        y = gpu_gemv(14, W, x)
        assert rel_err(y, ref) <= GEMV_TOL * 1e-2   # measured ~1e-6: the fp32 chain follows the reference's order
    pad = np.full((N, W.shape[1] + 210), 0x5A, np.uint8)
    pad[:, :W.shape[1]] = W
    assert np.array_equal(gpu_gemv(14, pad, x), gpu_gemv(14, W, x))


@pytest.mark.parametrize("nh,nkv,hd,past", [(32, 8, 128, 2100), (4, 2, 64, 19), (16, 2, 64, 63)])
def test_attn_decode_fused_q8_output_is_the_quantised_fp32_output(dev, nh, nkv, hd, past):
    """The decoder's internal attention entry also leaves the output as Q8 activation blocks for a Q4_K output
    projection: bit-identical to quantising the fp32 output with the stand-alone quantiser."""
    import ctypes as C
    from prometorch_amd import _lib
    L = _lib.load()
    fn = L.ptm_attn_decode_fused_q8
    vp = C.c_void_p
    fn.restype = C.c_int
    fn.argtypes = [vp] * 13 + [C.c_int, C.c_int, C.c_int, vp, C.c_int, C.c_float, C.c_float, C.c_int, C.c_int, C.c_int, vp]
    max_seq = ((past + 1 + 63) // 64 + 1) * 64
    r = synth.rng_for(49, nh, hd, past)
    kvd, qd = nkv * hd, nh * hd
    Kc = cu(r.standard_normal((max_seq, kvd), dtype=np.float32).astype(np.float16))
    Vc = cu(r.standard_normal((max_seq, kvd), dtype=np.float32).astype(np.float16))
    S = ops.flash_decode_num_splits(max_seq)
    pO, pL, pM = torch.empty(S * qd, device="cuda"), torch.empty(S * nh, device="cuda"), torch.empty(S * nh, device="cuda")
    table = ops.rope_table(max_seq, hd, 1e6).cuda()
    O = torch.empty(qd, device="cuda")
    q8 = torch.zeros(ops.q8_bytes(qd), dtype=torch.uint8, device="cuda")
    d_past = torch.full((1,), past, dtype=torch.int64, device="cuda")
    Q, K, V = cu(synth.make_x(r, qd) * 3), cu(synth.make_x(r, kvd) * 3), cu(synth.make_x(r, kvd))
    qw, kw = cu(1 + 0.1 * synth.make_x(r, hd)), cu(1 + 0.1 * synth.make_x(r, hd))
    p = lambda t: t.data_ptr()
    rc = fn(p(Q), p(K), p(V), p(qw), p(kw), p(Kc), p(Vc), p(O), p(q8), p(pO), p(pL), p(pM), p(table), nh, nkv, hd,
            p(d_past), max_seq, 1.0 / np.sqrt(hd), 1e-6, 0, 1, 0, None)
    assert rc == 0
    torch.cuda.synchronize()
    want = torch.zeros_like(q8)
    ops.launch_quantize_q8(O, want, qd)
    torch.cuda.synchronize()
    assert torch.equal(q8, want)


def test_gemv_random_shapes_vs_oracle(dev, po):
    """A fixed pseudo-random sweep over row counts, row lengths, formats and store modes: every launch rule (lane
    groups per row, blocks per pass, rolling passes, the one-workgroup-per-CU kernel, the plain formats) is met by
    shapes nobody picked by hand."""
    r = np.random.default_rng(20251125)
    worst = {}
    for case in range(48):
        qt = int(r.choice([12, 12, 14, 14, 13, 8, 6]))
        K = int(r.integers(1, 65)) * 256 if case % 3 else int(r.choice([256, 2560, 4096, 9728, 14336]))
        N = int(r.integers(1, 6000)) if case % 4 else int(r.choice([1, 31, 32, 33, 2560, 4096]))
        accumulate = bool(r.integers(0, 2))
        rr = synth.rng_for(36, case)
        W = synth.make_weight(rr, qt, N, K)
        x = synth.make_x(rr, K)
        ref = po.gemv(qt, W, x)
        if accumulate:
            y0 = synth.make_x(rr, N)
            y = gpu_gemv(qt, W, x, accumulate=True, y0=y0) - y0
            e = float(np.abs(y - ref).max() / max(np.sqrt((ref.astype(np.float64) ** 2).mean()), np.abs(y0).max(), 1e-30))
        else:
            e = rel_err(gpu_gemv(qt, W, x), ref)
        worst[qt] = max(worst.get(qt, 0.0), e)
        assert e <= GEMV_TOL * 1e-1, (case, qt, N, K, accumulate, e)
    print("worst rel err per type:", {k: "%.1e" % v for k, v in worst.items()})


def test_fused_argmax_of_nan_logits_publishes_a_row_inside_the_table(dev):
    """All-NaN logits (a NaN anywhere in the hidden state): no comparison is ever true; the fused lm_head tail must still
    publish an index inside [0, N), because the next captured step reads that row of the embedding table."""
    N, K = 1024, 256
    W = synth.make_weight(synth.rng_for(3), 14, N, K)
    Wd = torch.from_numpy(W).cuda()
    xd = torch.full((K,), float("nan"), device="cuda")
    logits = torch.zeros(N, device="cuda")
    idx = torch.full((1,), -7, dtype=torch.int64, device="cuda")
    ws = torch.empty(ops.argmax_workspace_bytes(N), dtype=torch.uint8, device="cuda")
    ops.q6k_gemv_argmax(Wd, xd, logits, K, N, W.shape[1], idx, ws)
    torch.cuda.synchronize()
    assert bool(torch.isnan(logits).all()) and 0 <= int(idx.item()) < N
