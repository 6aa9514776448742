"""CPU: the GGUF container reader (ptm_gguf_*) against files produced by this repository's writer: header,
metadata of every scalar kind, tensor table, alignment padding, data bytes; malformed files are refused with the
documented codes.  (Format per the GGUF description the reference's GGUFReader follows, torch/io/gguf_loader.h:386-630.)"""
import struct

import numpy as np
import pytest

from prometorch_amd import gguf
from prometorch_amd.testing import gguf_writer, synth
from prometorch_amd._lib import PtmError


def tiny_model(seed=7):
    cfg = dict(synth.TINY)
    layers = [synth.make_layer(seed, i, cfg) for i in range(cfg["n_layers"])]
    head = synth.make_head(seed, cfg)
    return cfg, layers, head


@pytest.mark.parametrize("alignment", [32, 64, 4096])
def test_roundtrip_tensor_table_and_bytes(tmp_path, alignment):
    r = synth.rng_for(3, alignment)
    q4 = synth.make_q4k(r, 6, 512)
    q6 = synth.make_q6k(r, 5, 256)
    f32 = r.standard_normal(7, dtype=np.float32)
    f16 = r.standard_normal((3, 8), dtype=np.float32).astype(np.float16)
    path = str(tmp_path / "t.gguf")
    gguf_writer.write_gguf(path, {"general.architecture": "qwen3", "qwen3.block_count": 2, "qwen3.rope.freq_base": 1e6,
                           "some.flag": True, "some.big": 2 ** 40, "some.list": [1, 2, 3], "some.names": ["x", "yy"]},
                    [("a.weight", gguf.Q4_K, [512, 6], q4), ("b.weight", gguf.Q6_K, [256, 5], q6),
                     ("c", gguf.F32, [7], f32), ("d", gguf.F16, [8, 3], f16), ("e", 2, [32], b"\0" * 18)],
                    alignment=alignment)
    with gguf.GGUFFile(path) as g:
        assert g.version == 3 and g.alignment == alignment and len(g) == 5
        assert g.get_string("general.architecture") == "qwen3"
        assert g.get_int("qwen3.block_count") == 2 and g.get_int("some.flag") == 1 and g.get_int("some.big") == 2 ** 40
        assert g.get_float("qwen3.rope.freq_base") == 1e6 and g.get_float("qwen3.block_count") == 2.0
        assert g.get_string("qwen3.block_count") is None and g.get_string("missing") is None
        with pytest.raises(PtmError) as e:
            g.get_int("missing")
        assert e.value.code == -10
        with pytest.raises(PtmError):
            g.get_int("some.list")      # arrays are not scalars
        a = g.tensor("a.weight")
        assert a["type"] == 12 and a["dims"] == [512, 6] and a["nbytes"] == q4.size
        assert np.array_equal(a["data"], q4.reshape(-1))
        b = g.tensor(1)
        assert b["name"] == "b.weight" and np.array_equal(b["data"], q6.reshape(-1))
        assert np.array_equal(g.tensor("c")["data"].view(np.float32), f32)
        assert np.array_equal(g.tensor("d")["data"].view(np.float16).reshape(3, 8), f16)
        assert g.tensor("e")["nbytes"] == -1   # Q4_0: listed, not sized
        with pytest.raises(PtmError) as e:
            g.tensor("nope")
        assert e.value.code == -10
        # the mapping base is page aligned and the data section starts at a multiple of the alignment
        offs = [g.tensor(i)["data"].ctypes.data for i in range(4)]
        assert all((o - offs[0]) % alignment == 0 for o in offs)


def test_model_file_has_the_reference_tensor_names(tmp_path):
    cfg, layers, head = tiny_model()
    path = str(tmp_path / "m.gguf")
    gguf_writer.model_to_gguf(path, cfg, layers, head)
    with gguf.GGUFFile(path) as g:
        assert g.get_int("qwen3.embedding_length") == cfg["hidden"]
        for name in ("token_embd.weight", "output_norm.weight", "blk.0.attn_q.weight", "blk.1.ffn_down.weight",
                     "blk.0.attn_q_norm.weight", "blk.1.attn_k_norm.weight", "blk.0.attn_output.weight"):
            g.tensor(name)
        qt, W = layers[1]["down"]
        t = g.tensor("blk.1.ffn_down.weight")
        assert t["type"] == qt and t["dims"] == [cfg["inter"], cfg["hidden"]] and np.array_equal(t["data"], W.reshape(-1))


def test_qwen2_model_file_carries_the_bias_vectors(tmp_path):
    """blk.N.attn_{q,k,v}.bias as F32 vectors, the names the reference looks up (gguf_model.h:6750-6753)."""
    from prometorch_amd.testing import synth
    cfg, layers, head = synth.tiny_qwen2(5)
    path = str(tmp_path / "q2.gguf")
    gguf_writer.model_to_gguf(path, cfg, layers, head, arch="qwen2")
    with gguf.GGUFFile(path) as g:
        assert g.get_string("general.architecture") == "qwen2"
        assert g.get_int("qwen2.attention.head_count_kv") == cfg["n_kv_heads"]
        for i in range(cfg["n_layers"]):
            for k, n in (("q", cfg["n_heads"] * cfg["head_dim"]), ("k", cfg["n_kv_heads"] * cfg["head_dim"]),
                         ("v", cfg["n_kv_heads"] * cfg["head_dim"])):
                t = g.tensor(f"blk.{i}.attn_{k}.bias")
                assert t["type"] == 0 and t["dims"] == [n]
                assert np.array_equal(t["data"].view(np.float32), layers[i][k + "_bias"])
        with pytest.raises(Exception):
            g.tensor("blk.0.attn_q_norm.weight")


def test_malformed_files_are_refused(tmp_path):
    good = str(tmp_path / "g.gguf")
    gguf_writer.write_gguf(good, {"general.architecture": "qwen3"}, [("c", gguf.F32, [8], np.zeros(8, np.float32))])
    raw = open(good, "rb").read()

    def code_of(data):
        p = str(tmp_path / "bad.gguf")
        open(p, "wb").write(data)
        with pytest.raises(PtmError) as e:
            gguf.GGUFFile(p)
        return e.value.code

    assert code_of(b"GGML" + raw[4:]) == -9                                  # magic
    assert code_of(raw[:4] + struct.pack("<I", 1) + raw[8:]) == -4            # version 1
    assert code_of(raw[:40]) == -9                                           # truncated inside the metadata
    assert code_of(raw[:-16]) == -9                                          # tensor data runs past the end of the file
    assert code_of(raw[:8] + struct.pack("<Q", 2 ** 40) + raw[16:]) == -9    # absurd tensor count
    assert code_of(b"short") == -8
    with pytest.raises(PtmError) as e:
        gguf.GGUFFile(str(tmp_path / "does_not_exist.gguf"))
    assert e.value.code == -8
    # version 2 is accepted
    v2 = str(tmp_path / "v2.gguf")
    gguf_writer.write_gguf(v2, {"general.architecture": "qwen3"}, [("c", gguf.F32, [8], np.zeros(8, np.float32))], version=2)
    with gguf.GGUFFile(v2) as g:
        assert g.version == 2
