"""GPU: the streaming-read kernel bench.py uses as its achievable ceiling (libptm_bench.so, not part of the product
library) really reads every byte."""
import numpy as np
import pytest
import torch

from prometorch_amd.testing import synth

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("nbytes", [16, 32768, 32768 + 16, (1 << 20) + 48, 14008320])
def test_stream_read_xor_matches_numpy(dev, nbytes):
    """per-32 KiB XORs equal numpy's"""
    import bench
    BL = bench.bench_lib()
    data = synth.rng_for(48, nbytes).integers(0, 256, nbytes, dtype=np.uint8)
    n = BL.bench_stream_read_partials(nbytes)
    assert n == (nbytes + 32767) // 32768
    d = torch.from_numpy(data).cuda()
    out = torch.full((n,), -1, dtype=torch.int32, device="cuda")
    s = torch.cuda.current_stream().cuda_stream
    assert BL.bench_stream_read_xor(d.data_ptr(), nbytes, out.data_ptr(), s) == 0
    torch.cuda.synchronize()
    words = np.zeros(n * 8192, np.uint32)
    words[:nbytes // 4] = data.view(np.uint32)
    want = np.bitwise_xor.reduce(words.reshape(n, 8192), axis=1)
    assert np.array_equal(out.cpu().numpy().view(np.uint32), want)
    assert BL.bench_stream_read_xor(d.data_ptr(), nbytes + 8, out.data_ptr(), s) == -1


@pytest.mark.parametrize("which,keys", [("prefill_gemm", ["us_with_row_conversion"]),
                                        ("prefill_attention", ["us_512_rows", "us_2048_rows"])])
def test_bench_single_kernel_mode(dev, which, keys):
    """`bench.py --only <kernel>` (the target of the counter passes quoted in profiles/) runs in a child process and prints
    one JSON line with positive times."""
    import json
    import os
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    p = subprocess.run([sys.executable, os.path.join(root, "bench.py"), "--only", which], capture_output=True, text=True, timeout=110)
    assert p.returncode == 0, p.stderr[-2000:]
    lines = [l for l in p.stdout.splitlines() if l.strip()]
    assert len(lines) == 1, p.stdout
    out = json.loads(lines[0])
    assert out["only"] == which
    for k in keys:
        assert 0.0 < out[k] < 1e5, out
