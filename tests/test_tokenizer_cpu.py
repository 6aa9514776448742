"""The tokenizer and chat template (host code of the library, no GPU) against the compiled reference's
GGUFTokenizer / apply_chat_template (torch/io/tokenizer.h:24-643, torch/io/gguf_model.h:4178-4236):
tests/golden/golden_tokenizer.json holds what the reference produced for the synthetic tokenizers of
prometorch_amd.synth -- written as GGUF files by this repository's writer and read by the reference's own
GGUFReader -- over prometorch_amd.synth.tokenizer_texts.  Bar: identical ids, identical decoded bytes."""
import base64
import json
import os

import numpy as np
import pytest

from prometorch_amd import gguf
from prometorch_amd.testing import gguf_writer, synth
from prometorch_amd._lib import PtmError
from prometorch_amd.tokenizer import Tokenizer, chat_template

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "golden_tokenizer.json")


@pytest.fixture(scope="module")
def golden_tok():
    with open(GOLDEN) as f:
        return json.load(f)


def from_gguf(kind, tmp_path):
    md = synth.make_tokenizer(kind)
    md["general.architecture"] = "qwen3"
    path = str(tmp_path / f"tok_{kind}.gguf")
    gguf_writer.write_gguf(path, md, [("dummy", 0, [4], np.zeros(4, np.float32))])
    f = gguf.GGUFFile(path)
    return md, f, Tokenizer.from_gguf(f)


@pytest.mark.parametrize("kind", ["gpt2", "llama", "greedy"])
def test_encode_decode_match_the_reference(kind, golden_tok, tmp_path):
    md, f, tok = from_gguf(kind, tmp_path)
    g = golden_tok["tokenizers"][kind]
    texts = synth.tokenizer_texts(kind)
    assert len(g["cases"]) == 2 * len(texts)
    assert tok.vocab_size == len(md["tokenizer.ggml.tokens"])
    for i, case in enumerate(g["cases"]):
        text = base64.b64decode(case["text"])
        assert text == texts[i // 2]
        ids = tok.encode(text, use_bos=case["use_bos"])
        assert ids == case["ids"], (kind, text, case["use_bos"])
        assert tok.decode(ids, skip_special=True) == base64.b64decode(case["decoded_skip"]), (kind, text)
        assert tok.decode(ids, skip_special=False) == base64.b64decode(case["decoded_all"]), (kind, text)
    want = [base64.b64decode(t) for t in g["token_bytes_from_minus1"]]
    got = [tok.token(i) for i in range(-1, tok.vocab_size + 1)]       # ids outside the vocabulary decode to nothing
    assert got == want
    tok.close()
    f.close()


@pytest.mark.parametrize("kind", ["gpt2", "llama"])
def test_lists_constructor_equals_gguf_constructor(kind, tmp_path):
    md, f, a = from_gguf(kind, tmp_path)
    b = Tokenizer.from_lists(md["tokenizer.ggml.tokens"], md.get("tokenizer.ggml.merges", []), md["tokenizer.ggml.model"],
                             bos_id=md["tokenizer.ggml.bos_token_id"], eos_id=md["tokenizer.ggml.eos_token_id"],
                             pad_id=md.get("tokenizer.ggml.padding_token_id", -1), unk_id=md.get("tokenizer.ggml.unknown_token_id", 0),
                             add_bos=md["tokenizer.ggml.add_bos_token"])
    assert a.special_ids() == b.special_ids()
    for text in synth.tokenizer_texts(kind):
        assert a.encode(text) == b.encode(text)
    # the reader hands the arrays over unchanged
    assert [t.decode() for t in f.get_array("tokenizer.ggml.tokens")] == md["tokenizer.ggml.tokens"]
    if kind == "llama":
        assert np.array_equal(f.get_array("tokenizer.ggml.scores"), np.zeros(len(md["tokenizer.ggml.tokens"]), np.float32))
    a.close(); b.close(); f.close()


def test_gpt2_round_trip_and_stray_continuation_bytes(tmp_path):
    md, f, tok = from_gguf("gpt2", tmp_path)
    # byte-level BPE loses nothing: every text without special tokens decodes to itself
    for text in synth.tokenizer_texts("gpt2"):
        if b"<" in text:
            continue
        assert tok.decode(tok.encode(text), skip_special=False) == text
    # continuation bytes that do not follow a letter (the reference's splitter does not return on these)
    for text in (b"\x80", b"1\x80\x81", b" \xbf!", b"?\x9f x", bytes(range(0x80, 0xc0))):
        assert tok.decode(tok.encode(text), skip_special=False) == text
    tok.close(); f.close()


def test_encode_reports_the_needed_size(tmp_path):
    import ctypes as C
    md, f, tok = from_gguf("gpt2", tmp_path)
    text = b"hello world, hello world"
    n = C.c_int64()
    small = (C.c_int32 * 2)()
    rc = tok.L.ptm_tokenizer_encode(tok.h, text, len(text), 0, small, 2, C.byref(n))
    assert rc == -6 and n.value == len(tok.encode(text, use_bos=False)) > 2
    tok.close(); f.close()


def test_chat_template_matches_the_reference(golden_tok):
    assert len(golden_tok["chat"]) >= 12
    for c in golden_tok["chat"]:
        got = chat_template(c["arch"], c["prompt"], model_name=c["name"], system=c["system"], no_think=c["no_think"])
        assert got.decode() == c["text"], c


def test_gguf_arrays_malformed(tmp_path):
    md = {"general.architecture": "qwen3", "a.strings": ["x", "", "yz"], "a.ints": [1, -2, 3], "a.floats": [0.5, 1.5]}
    path = str(tmp_path / "arr.gguf")
    gguf_writer.write_gguf(path, md, [])
    with gguf.GGUFFile(path) as f:
        assert f.get_array("a.strings") == [b"x", b"", b"yz"]
        assert list(f.get_array("a.ints")) == [1, -2, 3] and list(f.get_array("a.floats")) == [0.5, 1.5]
        with pytest.raises(PtmError):
            f.get_array("general.architecture")          # not an array
        with pytest.raises(PtmError):
            f.get_array("missing")
    raw = open(path, "rb").read()
    cut = raw[:raw.index(b"a.strings") + 9 + 4 + 4 + 8 + 8 + 1]   # file ends inside the second element's length field
    bad = str(tmp_path / "cut.gguf")
    open(bad, "wb").write(cut)
    with pytest.raises(PtmError):
        gguf.GGUFFile(bad)
