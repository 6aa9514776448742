"""CPU: the C-ABI library loads and exports every symbol include/ptm.h declares; host-side
argument validation returns error codes without touching a GPU."""
import ctypes as C
import os
import re

import numpy as np
import pytest

from conftest import ROOT
from prometorch_amd import _lib


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "ptm.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(ptm_[a-z0-9_]+)\s*\(", text)))


def test_library_built_and_exports_every_declared_symbol():
    assert os.path.exists(_lib.LIB_PATH), "libptm_hip.so is not built (python -m prometorch_amd.build)"
    raw = C.CDLL(_lib.LIB_PATH)
    names = declared_symbols()
    assert len(names) >= 40
    for n in names:
        assert hasattr(raw, n), f"{n} declared in ptm.h but not exported"
    assert set(names) == set(_lib.SIGNATURES), set(names) ^ set(_lib.SIGNATURES)


def test_shim_header_names_exist_in_abi():
    shim = open(os.path.join(ROOT, "include", "ptm_at_cuda_shim.h")).read()
    shim = re.sub(r"/\*.*?\*/", "", shim, flags=re.S)
    used = set(re.findall(r"\b(ptm_[a-z0-9_]+)\s*\(", shim)) - {"ptm_shim_context", "ptm_shim_set_context"}  # the shim's own
    assert used and used <= set(declared_symbols()), used - set(declared_symbols())


def test_shim_header_compiles_as_host_cxx(tmp_path):
    """Reference host code includes the shim in place of ATen/cuda/CUDAOps.h: it must be plain host C++."""
    import shutil
    import subprocess
    if not (shutil.which("g++") and os.path.isdir("/opt/rocm/include")):
        pytest.skip("no g++ / ROCm headers")
    src = tmp_path / "uses_shim.cpp"
    src.write_text(
        '#include "ptm_at_cuda_shim.h"\n'
        "void step(const void* w, const float* x, float* y, cudaStream_t s) {\n"
        "    at::cuda::launch_q4km_persistent_gemv(w, x, y, 2560, 9728, 1440, s);\n"
        "    at::cuda::launch_q6k_gemv(w, x, y, 2560, 1024, 2100);\n"
        "    at::cuda::launch_rms_norm(x, x, y, 1, 2560, 1e-6f, false, s);\n"
        "    at::cuda::launch_silu_mul(x, x, y, 9728, s);\n"
        "}\n")
    r = subprocess.run(["g++", "-std=c++17", "-fsyntax-only", "-Wall", "-Werror", "-D__HIP_PLATFORM_AMD__",
                        "-I/opt/rocm/include", "-I" + os.path.join(ROOT, "include"), str(src)],
                       capture_output=True, text=True)
    assert r.returncode == 0, r.stderr


def test_host_side_validation_codes():
    L = _lib.load()
    E_NULL, E_SHAPE, E_ALIGN, E_UNSUP = -1, -2, -3, -4
    assert L.ptm_q4k_gemv(None, None, None, 256, 4, 144, 0, None) == E_NULL
    assert L.ptm_q4k_gemv(16, 16, 16, 250, 4, 144, 0, None) == E_SHAPE       # K not a multiple of 256
    assert L.ptm_q4k_gemv(16, 16, 16, 256, 0, 144, 0, None) == E_SHAPE       # empty N
    assert L.ptm_q4k_gemv(16, 16, 16, 256, 4, 100, 0, None) == E_SHAPE       # stride < row bytes
    assert L.ptm_q4k_gemv(24, 16, 16, 256, 4, 144, 0, None) == E_ALIGN
    assert L.ptm_q4k_gemv(16, 16, 16, 65536, 4, 144 * 256, 0, None) == E_UNSUP
    assert L.ptm_q6k_gemv(16, 16, 16, 256, 4, 209, 0, None) == E_SHAPE
    assert L.ptm_q6k_gemv(17, 16, 16, 256, 4, 210, 0, None) == E_ALIGN
    assert L.ptm_quant_gemv(10, 16, 16, 16, 256, 4, 84, 0, None) == E_UNSUP   # Q2_K: not in the reference's dispatcher either
    assert L.ptm_quant_gemv(13, 16, 16, 16, 250, 4, 176, 0, None) == E_SHAPE  # Q5_K: K not a multiple of 256
    assert L.ptm_quant_gemv(13, 18, 16, 16, 256, 4, 176, 0, None) == E_ALIGN  # Q5_K blocks are read as dwords
    assert L.ptm_quant_gemv(8, 16, 16, 16, 48, 4, 68, 0, None) == E_SHAPE     # Q8_0: K not a multiple of 32
    assert L.ptm_quant_gemv(8, 17, 16, 16, 64, 4, 68, 0, None) == E_ALIGN
    assert L.ptm_quant_gemv(6, 16, 16, 16, 64, 4, 43, 0, None) == E_SHAPE     # Q5_0: stride below two 22-byte blocks
    assert [t for t in range(32) if L.ptm_quant_gemv_supported(t)] == [6, 8, 12, 13, 14]  # cpu_quant_gemv.h:1691-1694
    assert L.ptm_flash_decode(16, 16, 16, 16, 16, 16, 16, 32, 8, 96, 16, 128, 1.0, 1, None) == E_UNSUP
    assert L.ptm_flash_decode(16, 16, 16, 16, 16, 16, 16, 30, 8, 128, 16, 128, 1.0, 1, None) == E_SHAPE
    assert L.ptm_dequant_q4k(16, 16, 100, None) == E_SHAPE
    assert L.ptm_dequant_q4k(16, 16, 0, None) == 0                            # empty input is fine
    assert L.ptm_rms_norm(16, 16, 16, 2, 256, 1e-6, 0, 16, None) == E_SHAPE   # Q8 output only for one row
    assert L.ptm_strerror(E_SHAPE).decode().startswith("bad shape")
    assert L.ptm_q8_bytes(2560) == 2560 + 640
    assert L.ptm_flash_decode_num_splits(2176) == 34 and L.ptm_flash_decode_kv_chunk_size() == 64
    assert L.ptm_decode_create(None, None) == E_NULL
    # the qwen2 / gemma3 additions
    assert L.ptm_add_qkv_bias(16, 16, 16, 16, 16, None, 1, 256, 64, None) == E_NULL
    assert L.ptm_add_qkv_bias(16, 16, 16, 16, 16, 16, 1, 0, 64, None) == E_SHAPE
    assert L.ptm_add_qkv_bias(16, 16, 16, 16, 16, 16, 0, 256, 64, None) == 0            # no rows: nothing to do
    assert L.ptm_rms_norm_add(16, 16, None, 1, 256, 1e-6, 0, None) == E_NULL
    assert L.ptm_rms_norm_add(16, 16, 20, 1, 256, 1e-6, 0, None) == E_ALIGN            # rows are read as float4
    assert L.ptm_gelu_mul(16, None, 16, 8, None) == E_NULL and L.ptm_gelu_mul(16, 16, 16, -1, None) == E_SHAPE
    assert L.ptm_scale(None, 2.0, 8, None) == E_NULL and L.ptm_scale(16, 2.0, 0, None) == 0
    assert L.ptm_flash_decode_window(16, 16, 16, 16, None, 16, 16, 16, 32, 8, 96, 16, 128, 1.0, 1, 8, None) == E_UNSUP
    assert L.ptm_flash_decode_window(16, 16, 16, 16, 24, 16, 16, 16, 8, 4, 256, 16, 128, 1.0, 1, 8, None) == E_ALIGN  # Q8 copy
    assert L.ptm_prefill_attention_window(16, 16, 16, 16, 4, 4, 2, 96, 0, 16, 0.1, 0, 8, None) == E_UNSUP
    assert L.ptm_prefill_attention_window(16, 16, 16, 16, 4, 4, 2, 256, 14, 16, 0.1, 0, 8, None) == -6  # rows run past the cache
    assert L.ptm_attn_decode_fused_window(16, 16, 16, 16, None, 16, 16, 16, 16, 16, 16, 16, 8, 4, 256, 16, 128, 1.0, 1e-6, 0,
                                          1, 0, 8, None) == E_NULL                    # QK-norm weights: both or neither


def test_rope_table_host_matches_oracle(po):
    from prometorch_amd import ops
    t = ops.rope_table(40, 128, 1e6).numpy()
    for pos in (0, 1, 39):
        c, s = po.rope_tables(pos, 128, 1e6)
        assert np.array_equal(t[pos, :64].view(np.uint32), c.view(np.uint32))
        assert np.array_equal(t[pos, 64:].view(np.uint32), s.view(np.uint32))
    # linear position scaling, 256-wide heads
    t = ops.rope_table(70, 256, 1e6, 8.0).numpy()
    for pos in (0, 7, 69):
        c, s = po.rope_tables(pos, 256, 1e6, 8.0)
        assert np.array_equal(t[pos, :128].view(np.uint32), c.view(np.uint32))
        assert np.array_equal(t[pos, 128:].view(np.uint32), s.view(np.uint32))


def test_synth_generators_are_deterministic_and_in_range():
    from prometorch_amd.testing import synth
    a = synth.make_q4k(synth.rng_for(3), 4, 512)
    b = synth.make_q4k(synth.rng_for(3), 4, 512)
    assert np.array_equal(a, b) and a.shape == (4, 288)
    sc, mn = synth.unpack_scales_k4(a.reshape(-1, 144)[:, 4:16])
    assert sc.max() <= 63 and mn.max() <= 63
    w6 = synth.make_q6k(synth.rng_for(3), 4, 512).reshape(-1, 210)
    s8 = w6[:, 192:208].view(np.int8)
    assert s8.min() >= -32 and s8.max() <= 31
    d = w6[:, 208:210].copy().view(np.float16)
    assert np.all(d >= 0) and np.all(np.isfinite(d))
