"""GPU: ptm_q6k_gemv_argmax_noalloc (per-workgroup argmax partials in a device array inside the library, no workspace
argument, no allocation) gives exactly what ptm_q6k_gemv_argmax gives with a caller workspace - on two calls in a row that
share the array, the second with a smaller matrix - and refuses more rows than the array holds."""
import numpy as np
import pytest
import torch

from prometorch_amd import _lib, ops
from prometorch_amd.testing import synth

pytestmark = pytest.mark.gpu


def test_q6k_gemv_argmax_noalloc_matches_workspace_form_twice(dev, po):
    L = ops._L()
    s = torch.cuda.current_stream().cuda_stream
    max_rows = L.ptm_q6k_gemv_argmax_noalloc_max_rows()
    assert max_rows == 262144
    rng = synth.rng_for(41)
    keep = []
    for call, (N, K) in enumerate(((4096, 2560), (1000, 512))):   # the second call is smaller: stale partials lie behind it
        W = synth.make_weight(rng, 14, N, K)
        x = synth.make_x(rng, K)
        Wd, xd = torch.from_numpy(W).cuda(), torch.from_numpy(x).cuda()
        keep += [Wd, xd]
        want_logits = torch.zeros(N, device="cuda")
        want_idx = torch.full((1,), -1, dtype=torch.int64, device="cuda")
        ws = torch.empty(ops.argmax_workspace_bytes(N), dtype=torch.uint8, device="cuda")
        ops.q6k_gemv_argmax(Wd, xd, want_logits, K, N, W.shape[1], want_idx, ws)
        got_logits = torch.zeros(N, device="cuda")
        got_idx = torch.full((1,), -1, dtype=torch.int64, device="cuda")
        torch.cuda.synchronize()
        before = torch.cuda.memory_allocated()
        _lib.check(L.ptm_q6k_gemv_argmax_noalloc(Wd.data_ptr(), xd.data_ptr(), got_logits.data_ptr(), K, N, W.shape[1],
                                                 got_idx.data_ptr(), s), "q6k_gemv_argmax_noalloc")
        torch.cuda.synchronize()
        assert torch.cuda.memory_allocated() == before
        assert torch.equal(got_logits, want_logits), call                 # bit-exact: the same kernels
        assert int(got_idx.item()) == int(want_idx.item()), call
        ref = po.gemv(14, W, x)
        assert int(got_idx.item()) == int(np.argmax(ref)), call           # and the oracle's argmax
        # logits = NULL: argmax only
        got_idx.fill_(-1)
        _lib.check(L.ptm_q6k_gemv_argmax_noalloc(Wd.data_ptr(), xd.data_ptr(), None, K, N, W.shape[1], got_idx.data_ptr(), s),
                   "q6k_gemv_argmax_noalloc (no logits)")
        torch.cuda.synchronize()
        assert int(got_idx.item()) == int(want_idx.item()), call
    # beyond the array: refused on the host, nothing launched
    assert L.ptm_q6k_gemv_argmax_noalloc(16, 16, 16, 256, max_rows + 1, 210, 16, None) == -6
    assert L.ptm_q6k_gemv_argmax_noalloc(None, 16, 16, 256, 8, 210, 16, None) == -1


def test_q6k_gemv_argmax_noalloc_under_graph_capture(dev, po):
    """After ptm_q6k_gemv_argmax_noalloc_init() (symbol lookup and kernel attributes, once per device, outside capture) the
    entry point is legal under stream capture: captured once, replayed three times with other inputs written in between, every
    replay equal to the workspace form run eagerly on the same inputs.  A row long enough to need the raised LDS cap."""
    L = ops._L()
    assert L.ptm_q6k_gemv_argmax_noalloc_init() == 0
    rng = synth.rng_for(43)
    N, K = 1536, 16384                       # K * 4.25 B of staged activations: above the default 64 KB of dynamic LDS
    W = synth.make_weight(rng, 14, N, K)
    Wd = torch.from_numpy(W).cuda()
    xd = torch.zeros(K, device="cuda")
    got_logits = torch.zeros(N, device="cuda")
    got_idx = torch.full((1,), -1, dtype=torch.int64, device="cuda")
    want_logits = torch.zeros(N, device="cuda")
    want_idx = torch.full((1,), -1, dtype=torch.int64, device="cuda")
    ws = torch.empty(ops.argmax_workspace_bytes(N), dtype=torch.uint8, device="cuda")
    side = torch.cuda.Stream()
    g = torch.cuda.CUDAGraph()
    torch.cuda.synchronize()
    with torch.cuda.graph(g, stream=side):
        _lib.check(L.ptm_q6k_gemv_argmax_noalloc(Wd.data_ptr(), xd.data_ptr(), got_logits.data_ptr(), K, N, W.shape[1],
                                                 got_idx.data_ptr(), torch.cuda.current_stream().cuda_stream),
                   "q6k_gemv_argmax_noalloc under capture")
    for rep in range(3):
        x = synth.make_x(rng, K)
        xd.copy_(torch.from_numpy(x))
        torch.cuda.synchronize()
        g.replay()
        torch.cuda.synchronize()
        ops.q6k_gemv_argmax(Wd, xd, want_logits, K, N, W.shape[1], want_idx, ws)
        torch.cuda.synchronize()
        assert torch.equal(got_logits, want_logits), rep
        assert int(got_idx.item()) == int(want_idx.item()), rep
        if rep == 0:
            assert int(got_idx.item()) == int(np.argmax(po.gemv(14, W, x)))
