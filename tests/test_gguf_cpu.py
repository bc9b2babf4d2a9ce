"""GGUF reader (src/gguf.cpp, src/loader.cpp:213-541), checked without a GPU: the
numpy restatement in oracle/gguf_oracle.py against the compiled reference
(oracle/_ref, where built) and a hand-assembled file; the product's host-side
reader (lpp_gguf_*) against the restatement."""
import struct
import sys
from pathlib import Path

import numpy as np
import pytest

sys.path.insert(0, str(Path(__file__).resolve().parent.parent / "oracle"))

import gguf_oracle as go  # noqa: E402
import gguf_writer as gw  # noqa: E402
import oracle_binding as ob  # noqa: E402
from lighterpp_amd import Gguf, Shape, capi, synth_tensor  # noqa: E402

CASES = {
    # name: (Shape, f16 matrices, f16 embedding in the file, writer options)
    "f32_tied": (Shape(64, 160, 2, 8, 2, 96, 48, 10000.0, fp16=False, tied=True), False, False, {}),
    "f32_untied_mha_defaults": (Shape(48, 96, 3, 4, 4, 70, 32, 10000.0, fp16=False, tied=False), False, False,
                                {"with_kv_heads": False, "with_rope": False, "noise": False}),
    "f16_tied_llama3like": (Shape(128, 256, 2, 16, 4, 200, 64, 500000.0, fp16=True, tied=True), True, True, {}),
    "f16_untied_f32_embedding": (Shape(64, 192, 2, 4, 2, 120, 40, 500000.0, fp16=True, tied=False), True, False,
                                 {"arch": "mistral"}),
    "context_capped": (Shape(32, 64, 1, 4, 2, 50, 16384, 10000.0, fp16=False, tied=True), False, False,
                       {"context": 131072}),
}


def make(tmp_path, name):
    shape, f16m, f16e, opts = CASES[name]
    w = {t: synth_tensor(shape, t, 41) for t in range(12)}
    path = tmp_path / f"{name}.gguf"
    gw.write_gguf(path, gw.llama_kv(shape, **opts), gw.llama_tensors(shape, w, f16m, f16e))
    return shape, w, path


def expected_f32(shape, w, f16e):
    """What a correct reader must end up with, from the arrays the file was written from."""
    out = []
    for t in range(12):
        a = np.ascontiguousarray(w[t])
        a = capi.f16_to_f32(a) if a.dtype == np.uint16 else a.astype(np.float32)
        out.append(a.reshape(-1))
    if f16e:  # the embedding went through binary16 in the file
        out[0] = out[0].astype(np.float16).astype(np.float32)
    if shape.tied:
        out[11] = out[0]
    return out


@pytest.mark.parametrize("name", list(CASES))
def test_oracle_reads_what_was_written_and_what_the_reference_reads(name, tmp_path):
    shape, w, path = make(tmp_path, name)
    f16e = CASES[name][2]
    buf = path.read_bytes()
    g = go.parse(buf)
    cfg = go.extract_config(buf, g)
    want_seq = min(CASES[name][3].get("context", shape.seq_len), 16384)
    assert (cfg["dim"], cfg["hidden_dim"], cfg["n_layers"], cfg["n_heads"], cfg["n_kv_heads"], cfg["vocab_size"],
            cfg["seq_len"]) == (shape.dim, shape.hidden_dim, shape.n_layers, shape.n_heads, shape.n_kv_heads,
                                shape.vocab_size, want_seq)
    assert cfg["rope_base"] == np.float32(shape.rope_base) and cfg["fp16"] == shape.fp16
    arrays, tied = go.stacked_weights(buf, g, cfg)
    assert tied == shape.tied
    for t, (got, want) in enumerate(zip(arrays, expected_f32(shape, w, f16e))):
        assert np.array_equal(got.view(np.uint32), want.view(np.uint32)), f"tensor {t}"
    if ob.have_ref():
        r = ob.ref_gguf_load(path)
        assert r is not None
        rcfg, rarrays, rtied = r
        for k in ("dim", "hidden_dim", "n_layers", "n_heads", "n_kv_heads", "vocab_size", "seq_len", "fp16"):
            assert rcfg[k] == cfg[k], k
        assert rcfg["rope_base"] == cfg["rope_base"] and rtied == tied
        for t in range(12):
            assert np.array_equal(rarrays[t].view(np.uint32), arrays[t].view(np.uint32)), f"tensor {t} vs reference"


def test_oracle_on_a_hand_assembled_file():
    """Every offset worked out by hand: 24-byte header, one pair, one 1-d F32 tensor."""
    kv = gw.gstr("general.architecture") + struct.pack("<I", go.STRING) + gw.gstr("llama")  # 28 + 4 + 13 = 45 bytes
    info = gw.gstr("output_norm.weight") + struct.pack("<IQIQ", 1, 3, go.GGML_F32, 0)      # 26 + 24 = 50 bytes
    pre = struct.pack("<IIQQ", 0x46554747, 3, 1, 1) + kv + info                              # 24 + 45 + 50 = 119
    assert len(pre) == 119
    buf = pre + b"\0" * 9 + np.array([1.0, 2.0, 3.0], np.float32).tobytes()                  # data at 128
    g = go.parse(buf)
    assert g["data_start"] == 128 and g["meta"]["general.architecture"] == (go.STRING, 24 + 28 + 4)
    assert g["tensors"]["output_norm.weight"] == (go.GGML_F32, (3,), 0)
    assert go.tensor(buf, g, "output_norm.weight")[1].tolist() == [1.0, 2.0, 3.0]
    for bad in (b"XXXX" + buf[4:], buf[:4] + struct.pack("<I", 1) + buf[8:], buf[:4] + struct.pack("<I", 4) + buf[8:]):
        with pytest.raises(go.GgufError):
            go.parse(bad)


def test_a_key_of_another_type_reads_as_missing(tmp_path):
    """gguf.cpp:311-336: a getter answers only for its own value type; rope.freq_base written as a
    double falls back to 10000, head_count_kv written as u64 falls back to head_count."""
    shape = Shape(32, 64, 1, 4, 4, 30, 16, 10000.0, fp16=False, tied=True)
    w = {t: synth_tensor(shape, t, 2) for t in range(12)}
    kv = gw.llama_kv(shape, with_kv_heads=False, with_rope=False, noise=False)
    kv.insert(1, ("llama.rope.freq_base", gw.F64, 500000.0))
    kv.insert(1, ("llama.attention.head_count_kv", gw.U64, 2))
    path = tmp_path / "odd.gguf"
    gw.write_gguf(path, kv, gw.llama_tensors(shape, w, False))
    buf = path.read_bytes()
    cfg = go.extract_config(buf, go.parse(buf))
    assert cfg["rope_base"] == np.float32(10000.0) and cfg["n_kv_heads"] == 4
    g = Gguf(path)
    assert g.config.rope_base == 10000.0 and g.config.n_kv_heads == 4
    if ob.have_ref():
        rcfg = ob.ref_gguf_load(path)[0]
        assert rcfg["rope_base"] == np.float32(10000.0) and rcfg["n_kv_heads"] == 4


@pytest.mark.parametrize("name", list(CASES))
def test_product_reader_agrees_with_the_oracle(name, tmp_path):
    shape, w, path = make(tmp_path, name)
    buf = path.read_bytes()
    og = go.parse(buf)
    cfg = go.extract_config(buf, og)
    g = Gguf(path)
    c = g.config
    assert (c.dim, c.hidden_dim, c.n_layers, c.n_heads, c.n_kv_heads, c.vocab_size, c.seq_len) == \
           (cfg["dim"], cfg["hidden_dim"], cfg["n_layers"], cfg["n_heads"], cfg["n_kv_heads"], cfg["vocab_size"],
            cfg["seq_len"])
    assert np.float32(c.rope_base) == cfg["rope_base"]
    assert (c.weight_precision == capi.WEIGHT_FP16) == cfg["fp16"]
    for name_t in og["tensors"]:
        ty, want = go.tensor(buf, og, name_t)
        got = g.tensor(name_t)
        assert got.dtype == want.dtype and np.array_equal(got, want), name_t
    assert g.has_tensor("output.weight") == (not shape.tied)
    g.close()


def test_product_reader_rejects_broken_files(tmp_path):
    shape, w, path = make(tmp_path, "f32_tied")
    buf = path.read_bytes()

    def refuses(name, data, match=None):
        p = tmp_path / name
        p.write_bytes(data)
        with pytest.raises(capi.LppError, match=match):
            Gguf(p)

    with pytest.raises(capi.LppError):
        Gguf(tmp_path / "missing.gguf")
    refuses("magic.gguf", b"GGML" + buf[4:], "not a GGUF")
    refuses("version.gguf", buf[:4] + struct.pack("<I", 1) + buf[8:], "version")
    refuses("header.gguf", buf[:20])
    refuses("cut_meta.gguf", buf[:200], "truncated|past the end")
    refuses("cut_data.gguf", buf[:-64], "past the end")
    # a file without the vocabulary cannot give a config
    kv = [e for e in gw.llama_kv(shape, noise=False) if e[0] != "tokenizer.ggml.tokens"]
    p = tmp_path / "novocab.gguf"
    gw.write_gguf(p, kv, gw.llama_tensors(shape, w, False))
    with pytest.raises(capi.LppError, match="tokenizer.ggml.tokens"):
        Gguf(p).config
    if ob.have_ref():
        assert ob.ref_gguf_load(p) is None
