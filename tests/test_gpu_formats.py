"""GPU: the GEMV dispatcher's other block formats (Q5_K, Q8_0, Q5_0; cpu_quant_gemv.h:1635-1694) through the C ABI
against the CPU oracle and the compiled reference's golden outputs.  Bars as for Q4_K / Q6_K: GEMV within 1e-3 of
rms(y) (measured ~1e-6: fp32 accumulation, exact quants), dequantised values bit-exact."""
import os

import numpy as np
import pytest
import torch

from conftest import GOLDEN_DIR, bits
from prometorch_amd import ops
from prometorch_amd.testing import synth
from prometorch_amd._lib import PtmError
from test_gpu_parity import GEMV_TOL, cu, gpu_gemv, rel_err

pytestmark = pytest.mark.gpu

GOLDEN_CASES = [(13, 24, 512), (13, 3, 2560), (8, 24, 512), (8, 5, 96), (6, 24, 512), (6, 7, 32)]


@pytest.fixture(scope="module")
def golden_formats():
    return np.load(os.path.join(GOLDEN_DIR, "golden_formats.npz"))


@pytest.mark.parametrize("qt,N,K", GOLDEN_CASES)
def test_other_formats_gemv_vs_reference_golden(dev, seeds, golden_formats, qt, N, K):
    r = synth.rng_for(seeds["blocks"], qt, N, K)
    W = synth.make_weight(r, qt, N, K)
    x = synth.make_x(r, K)
    e = rel_err(gpu_gemv(qt, W, x), golden_formats["y_%d_%d_%d" % (qt, N, K)])
    print(qt, N, K, "rel err vs the compiled reference", e)
    assert e <= GEMV_TOL * 1e-2


@pytest.mark.parametrize("qt,N,K", [(13, 33, 512), (13, 300, 2560), (13, 64, 9728), (13, 1, 256), (8, 33, 512),
                                    (8, 100, 4096), (8, 7, 96), (8, 2, 32), (6, 33, 512), (6, 5, 32), (6, 100, 4096),
                                    (13, 1000, 4096), (8, 1000, 2560)])
def test_other_formats_gemv_shapes_vs_oracle(dev, po, qt, N, K):
    r = synth.rng_for(35, qt, N, K)
    W = synth.make_weight(r, qt, N, K)
    x = synth.make_x(r, K)
    ref = po.gemv(qt, W, x)
    assert rel_err(gpu_gemv(qt, W, x), ref) <= GEMV_TOL * 1e-2
    # accumulate, and rows padded to a wider stride (a row-slice view of a wider tensor)
    y0 = synth.make_x(r, N)
    ya = gpu_gemv(qt, W, x, accumulate=True, y0=y0)
    assert np.abs((ya - y0) - ref).max() <= 1e-5 * max(np.abs(y0).max(), np.abs(ref).max())
    pad_by = {13: 176, 8: 34, 6: 22}[qt] * 2 + {13: 4, 8: 2, 6: 2}[qt]
    pad = np.full((N, W.shape[1] + pad_by), 0xA5, np.uint8)
    pad[:, :W.shape[1]] = W
    assert np.array_equal(gpu_gemv(qt, pad, x), gpu_gemv(qt, W, x))


@pytest.mark.parametrize("qt,N,K", [(13, 24, 512), (13, 3, 2560), (8, 24, 512), (8, 5, 96)])
def test_other_formats_dequant_bit_exact(dev, po, seeds, golden_formats, qt, N, K):
    r = synth.rng_for(seeds["blocks"], qt, N, K)
    W = synth.make_weight(r, qt, N, K)
    out = torch.empty(N * K, device="cuda")
    (ops.dequant_q5k if qt == 13 else ops.dequant_q8_0)(cu(W), out, N * K)
    torch.cuda.synchronize()
    got = out.cpu().numpy()
    assert np.array_equal(bits(got), bits(golden_formats["dq_%d_%d_%d" % (qt, N, K)]))
    assert np.array_equal(bits(got), bits(po.dequant(qt, W)))


def test_dispatcher_types_and_argument_errors(dev):
    assert [t for t in range(32) if ops.quant_gemv_supported(t)] == [6, 8, 12, 13, 14]
    x = torch.zeros(256, device="cuda")
    y = torch.full((4,), 7.0, device="cuda")
    W = torch.zeros(4 * 176, dtype=torch.uint8, device="cuda")
    with pytest.raises(PtmError) as e:
        ops.quant_gemv(10, W, x, y, 256, 4, 84)          # Q2_K: the reference's dispatcher does nothing either
    assert e.value.code == -4
    torch.cuda.synchronize()
    assert float(y.sum()) == 28.0                        # and nothing was launched
    with pytest.raises(PtmError):
        ops.quant_gemv(13, W, x, y, 256, 4, 100)         # stride below one super-block
    with pytest.raises(PtmError):
        ops.dequant_q5k(W, y, 100)                       # not a whole number of blocks
    with pytest.raises(PtmError):
        ops.dequant_q8_0(W, y, 48)


@pytest.mark.parametrize("N,K,accumulate", [(96, 2560, False), (5, 256, True), (1000, 4096, False)])
def test_q4k_fp32_activation_gemv_vs_oracle(dev, po, seeds, N, K, accumulate):
    """ptm_q4k_gemv_f32act: Q4_K with fp32 activations (the reference's scalar kernel, cpu_quant_gemv.h:689-767) against
    the oracle's restatement of it, which golden_q4k_f32act.npz pins to the compiled reference."""
    from prometorch_amd import _lib
    r = synth.rng_for(seeds["blocks"], 31, N)
    W = synth.make_q4k(r, N, K)
    x = synth.make_x(r, K)
    want = po.gemv(12, W, x, "f32")
    y0 = synth.make_x(r, N)
    Wd, xd = torch.from_numpy(W).cuda(), torch.from_numpy(x).cuda()
    y = torch.from_numpy(y0.copy()).cuda()
    _lib.check(ops._L().ptm_q4k_gemv_f32act(Wd.data_ptr(), xd.data_ptr(), y.data_ptr(), K, N, W.shape[1], int(accumulate),
                                            torch.cuda.current_stream().cuda_stream), "q4k_gemv_f32act")
    torch.cuda.synchronize()
    got = y.cpu().numpy() - (y0 if accumulate else 0)
    rms = np.sqrt((want.astype(np.float64) ** 2).mean())
    assert np.abs(got - want).max() / rms < (1e-3 if not accumulate else 1e-3 + 1e-6 * np.abs(y0).max() / rms)
    assert np.abs(got - want).max() / rms < 2e-5 or accumulate   # measured ~1e-6: only the summation order differs
