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
