"""CPU: the oracle's Q5_K / Q8_0 / Q5_0 functions (the GEMV dispatcher's other formats, cpu_quant_gemv.h:1635-1688)
against the compiled reference's outputs in golden_formats.npz (bit-exact) and against closed forms written here
independently in numpy (block layouts of gguf_dequant.h:237-255, :348-388; Q5_0 as cpu_quant_gemv.h:1606-1624)."""
import os

import numpy as np
import pytest

from conftest import GOLDEN_DIR, bits
from prometorch_amd.testing import synth

CASES = [(13, 24, 512), (13, 3, 2560), (8, 24, 512), (8, 5, 96), (6, 24, 512), (6, 7, 32)]


@pytest.fixture(scope="module")
def golden_formats():
    return np.load(os.path.join(GOLDEN_DIR, "golden_formats.npz"))


def case_inputs(seeds, qt, N, K):
    r = synth.rng_for(seeds["blocks"], qt, N, K)
    return synth.make_weight(r, qt, N, K), synth.make_x(r, K)


def f16(b):
    return np.ascontiguousarray(b).view(np.float16).astype(np.float32)


def numpy_dequant(qt, W, K):
    """Closed-form dequantisation of every row, float32 arithmetic in the reference's order."""
    N = W.shape[0]
    if qt == 8:
        blk = W.reshape(N, K // 32, 34)
        d = f16(blk[:, :, 0:2]).reshape(N, K // 32, 1)
        return (d * blk[:, :, 2:].view(np.int8).astype(np.float32)).reshape(N, K)
    if qt == 6:
        blk = W.reshape(N, K // 32, 22)
        d = f16(blk[:, :, 0:2]).reshape(N, K // 32, 1)
        qh = np.ascontiguousarray(blk[:, :, 2:6]).view(np.uint32).reshape(N, K // 32, 1)
        j = np.arange(16, dtype=np.uint32)
        lo = (blk[:, :, 6:] & 0xF).astype(np.int32) | (((qh >> j) & 1).astype(np.int32) << 4)
        hi = (blk[:, :, 6:] >> 4).astype(np.int32) | (((qh >> (j + 16)) & 1).astype(np.int32) << 4)
        q = np.concatenate([lo, hi], axis=2) - 16
        return (d * q.astype(np.float32)).reshape(N, K)
    blk = W.reshape(N, K // 256, 176)
    d, dmin = f16(blk[:, :, 0:2]), f16(blk[:, :, 2:4])
    s = blk[:, :, 4:16].astype(np.int32)
    sc = np.empty(blk.shape[:2] + (8,), np.int32)
    mn = np.empty_like(sc)
    for jj in range(8):   # get_scale_min_k4
        if jj < 4:
            sc[..., jj], mn[..., jj] = s[..., jj] & 63, s[..., jj + 4] & 63
        else:
            sc[..., jj] = (s[..., jj + 4] & 0xF) | ((s[..., jj - 4] >> 6) << 4)
            mn[..., jj] = (s[..., jj + 4] >> 4) | ((s[..., jj] >> 6) << 4)
    qh, qs = blk[:, :, 16:48], blk[:, :, 48:176].reshape(N, K // 256, 4, 32)
    out = np.empty((N, K // 256, 8, 32), np.float32)
    for sb in range(8):
        pair, hi = sb >> 1, sb & 1
        nib = (qs[:, :, pair] >> 4) if hi else (qs[:, :, pair] & 0xF)
        q = nib.astype(np.float32) + np.where((qh >> (2 * pair + hi)) & 1, np.float32(16), np.float32(0))
        ds = (d[:, :, 0] * sc[..., sb].astype(np.float32))[..., None]
        ms = (dmin[:, :, 0] * mn[..., sb].astype(np.float32))[..., None]
        out[:, :, sb] = ds * q - ms
    return out.reshape(N, K)


@pytest.mark.parametrize("qt,N,K", CASES)
def test_other_formats_vs_reference_and_closed_form(po, seeds, golden_formats, qt, N, K):
    W, x = case_inputs(seeds, qt, N, K)
    y = po.gemv(qt, W, x)
    assert np.array_equal(bits(y), bits(golden_formats["y_%d_%d_%d" % (qt, N, K)]))
    dq = numpy_dequant(qt, W, K)
    if qt != 6:
        got = po.dequant(qt, W).reshape(N, K)
        assert np.array_equal(bits(got), bits(golden_formats["dq_%d_%d_%d" % (qt, N, K)].reshape(N, K)))
        assert np.array_equal(bits(got), bits(dq))
    want = dq.astype(np.float64) @ x.astype(np.float64)
    assert np.abs(y - want).max() <= 3e-6 * np.sqrt((want ** 2).mean())


def test_other_formats_zero_and_extreme_blocks(po):
    """d = 0 blocks give exact zeros; the largest quants and scales stay finite."""
    x = np.ones(256, np.float32)
    z = np.zeros((1, 176), np.uint8)
    z[0, 16:] = 0xFF
    assert po.gemv(13, z, x)[0] == 0.0
    big = np.full((1, 8 * 34), 0x7F, np.uint8)
    big[0].reshape(8, 34)[:, 0:2] = np.array([0x7BFF], np.uint16).view(np.uint8)   # d = 65504
    y = po.gemv(8, big, x)
    assert np.isfinite(y[0]) and y[0] == np.float32(65504.0 * 127 * 256)
