"""Tokenizer (src/tokenizer.cpp, gguf_init_tokenizer of src/loader.cpp): the Python
restatement in oracle/tokenizer_oracle.py against the compiled reference (a fresh
copy of oracle/_ref per vocabulary, where built) and hand-worked cases; the
product's lpp_tokenizer_* against the restatement.  No GPU involved."""
import struct
import sys
from pathlib import Path

import numpy as np
import pytest

sys.path.insert(0, str(Path(__file__).resolve().parent.parent / "oracle"))

import gguf_writer as gw  # noqa: E402
import oracle_binding as ob  # noqa: E402
import tokenizer_oracle as to  # noqa: E402
from lighterpp_amd import Gguf, Shape, Tokenizer, capi, synth_tensor  # noqa: E402

SP = "▁".encode()   # SentencePiece space marker
G = "Ġ".encode()    # byte-pair space marker
NL = "Ċ".encode()   # byte-pair newline marker


def sentencepiece_vocab():
    """(strings, scores): specials, byte tokens for a few bytes, letters, merges with scores that make
    the merge order matter, duplicates, a malformed byte token, an over-long entry."""
    v = [b"<unk>", b"<s>", b"</s>"]
    v += [b"<0x%02X>" % b for b in (0x0A, 0x21, 0xC3, 0xA9, 0x00, 0x7A)]
    v += [SP] + [bytes([c]) for c in b"abcdehlorw,"]
    merges = [(b"he", -1.0), (b"ll", -2.0), (b"hel", -3.0), (b"lo", -1.5), (b"hello", -0.5), (SP + b"hello", -0.1),
              (b"wo", -4.0), (b"or", -3.5), (b"wor", -0.2), (b"ld", -6.0), (b"world", -0.3), (SP + b"w", -5.0),
              (b"ab", -1.0), (b"bc", -1.0), (b"abc", -9.0), (SP + SP, -7.0)]
    v += [m for m, _ in merges]
    scores = [0.0] * (len(v) - len(merges)) + [s for _, s in merges]
    v += [b"he", b"<0x1G>", b"x" * 300, b"<|weird|>", b"<>"]       # duplicate of an earlier entry (the later id wins)
    scores += [-0.05, 0.0, 0.0, 0.0, 0.0]
    return v, scores


def write_tokenizer_file(path, vocab, scores, max_len=None):
    with open(path, "wb") as f:
        f.write(struct.pack("<i", max_len if max_len is not None else max(len(s) for s in vocab)))
        for s, sc in zip(vocab, scores):
            f.write(struct.pack("<fi", sc, len(s)) + s)


TEXTS = [b"hello world", b"hello", b"", b" ", b"  hello", b"abc", b"abcabc", b"held", b"lol, world!", b"caf\xc3\xa9",
         b"zebra", b"hello\nworld", b"hellohello world world", b"wor ld", b"q"]


def test_hand_worked_encodings():
    v, s = sentencepiece_vocab()
    t = to.Tok(to.SENTENCEPIECE, v, s, 5)
    ids = {x: i for i, x in enumerate(v)}
    # "<s>" is entry 1 -> BOS; " hello" merges all the way to the single entry "▁hello"
    assert to.encode(t, b"hello") == [1, ids[SP + b"hello"]]
    # "abc": "ab" and "bc" score the same, the leftmost pair merges first; "abc" is then reachable from (ab, c)
    assert to.encode(t, b"abc") == [1, ids[SP], ids[b"abc"]]
    # '!' has no entry of its own: its byte token stands in; 'z' likewise; 'q' has neither and is dropped
    assert to.encode(t, b"!")[-1] == ids[b"<0x21>"]
    assert to.encode(t, b"q") == [1, ids[SP]]
    # decode: marker -> blank, byte token -> byte, other specials -> nothing, sscanf's leniency, 255-byte cut
    assert to.decode(t, ids[SP + b"hello"]) == b" hello"
    assert to.decode(t, ids[b"<0x0A>"]) == b"\n" and to.decode(t, ids[b"</s>"]) == b"" and to.decode(t, ids[b"<>"]) == b""
    assert to.decode(t, ids[b"<0x1G>"]) == b"\x01" and to.decode(t, ids[b"<0x00>"]) == b""
    assert to.decode(t, ids[b"x" * 300]) == b"x" * 255


def check_product_against_oracle(tok: Tokenizer, t: to.Tok, texts):
    assert (tok.vocab_size, tok.kind) == (len(t.vocab), t.kind)
    for i in range(len(t.vocab)):
        assert tok.decode(i) == to.decode(t, i), i
    for text in texts:
        if b"\0" in text:
            continue
        assert tok.encode(text) == to.encode(t, text), text
    assert tok.encode(b"hello world", max_tokens=2) == to.encode(t, b"hello world", 2)
    with pytest.raises(capi.LppError):
        tok.decode(len(t.vocab))
    with pytest.raises(capi.LppError):
        tok.decode(-1)


def check_reference_against_oracle(lib, h, t: to.Tok, texts):
    assert lib.ref_tokenizer_kind(h) == t.kind and lib.ref_tokenizer_vocab_size(h) == len(t.vocab)
    assert lib.ref_tokenizer_max_token_len(h) == t.max_token_len
    for i in range(len(t.vocab)):
        assert lib.ref_decode(h, i) == to.decode(t, i), i
        assert lib.ref_tokenizer_score(h, i) == np.float32(t.scores[i])
    for text in texts:
        want = to.encode(t, text)
        if not want:
            continue  # the reference's merge loop underflows on an empty list
        assert ob.ref_encode(lib, h, text) == want, text


def test_tokenizer_file(tmp_path):
    v, s = sentencepiece_vocab()
    path = tmp_path / "tokenizer.bin"
    write_tokenizer_file(path, v, s, max_len=7)
    t = to.load_file(path.read_bytes(), len(v))
    assert t.vocab == v and t.max_token_len == 7
    if ob.have_ref():
        lib = ob.fresh_ref(tmp_path)
        check_reference_against_oracle(lib, lib.ref_tokenizer_load(str(path).encode(), len(v)), t, TEXTS)
    tok = Tokenizer.load(path, len(v))
    assert tok.max_token_len == 7
    check_product_against_oracle(tok, t, TEXTS)
    # fewer entries than the file holds is what the caller asked for; more is an error
    assert Tokenizer.load(path, 10).vocab_size == 10
    with pytest.raises(capi.LppError, match="file ends"):
        Tokenizer.load(path, len(v) + 1)
    with pytest.raises(capi.LppError):
        Tokenizer.load(tmp_path / "missing.bin", 3)


def bpe_vocab():
    v = [b"<|begin_of_text|>", b"<|end_of_text|>", G, NL] + [bytes([c]) for c in b"helowrd!"]
    merges = [(b"he", 5.0), (b"ll", 4.0), (b"llo", 3.5), (b"hello", 3.0), (G + b"w", 2.5), (G + b"wo", 2.0), (b"rl", 1.0),
              (b"rld", 0.9), (G + b"world", 0.5), (G + b"hello", 6.0), (b"h\0idden", 0.0)]
    return v + [m for m, _ in merges], [0.0] * len(v) + [s for _, s in merges]


@pytest.mark.parametrize("model,with_scores", [("gpt2", True), ("llama", True), (None, False), ("gpt2", False)])
def test_tokenizer_from_gguf(model, with_scores, tmp_path):
    v, s = bpe_vocab() if model == "gpt2" else sentencepiece_vocab()
    shape = Shape(32, 64, 1, 4, 2, len(v), 16, 10000.0, fp16=False, tied=True)
    w = {t: synth_tensor(shape, t, 2) for t in range(12)}
    kv = [e for e in gw.llama_kv(shape, noise=False) if e[0] != "tokenizer.ggml.tokens"]
    if model is not None:
        kv.append(("tokenizer.ggml.model", gw.STRING, model))
    kv.append(("tokenizer.ggml.tokens", gw.ARRAY, (gw.STRING, v)))
    if with_scores:
        kv.append(("tokenizer.ggml.scores", gw.ARRAY, (gw.F32, s)))
    else:
        kv.append(("tokenizer.ggml.scores", gw.ARRAY, (gw.F32, s[:3])))  # wrong count: ignored, zeros instead
    path = tmp_path / "m.gguf"
    gw.write_gguf(path, kv, gw.llama_tensors(shape, w, False))
    t = to.from_gguf(model, v, s if with_scores else None)
    texts = [b"hello world", b"hello", b"world!", b"hello\nworld", b" ", b"held", b"abc"]
    if ob.have_ref():
        lib = ob.fresh_ref(tmp_path)
        check_reference_against_oracle(lib, lib.ref_tokenizer_from_gguf(str(path).encode()), t, texts)
    g = Gguf(path)
    tok = Tokenizer.from_gguf(g)
    g.close()
    assert tok.max_token_len == t.max_token_len
    check_product_against_oracle(tok, t, texts)


def test_bpe_hand_worked():
    v, s = bpe_vocab()
    t = to.from_gguf("gpt2", v, s)
    ids = {x: i for i, x in enumerate(t.vocab)}
    assert to.encode(t, b"hello world") == [ids[b"<|begin_of_text|>"], ids[G + b"hello"], ids[G + b"world"]]
    assert to.decode(t, ids[G + b"world"]) == b" world" and to.decode(t, ids[NL]) == b"\n"
    assert to.decode(t, ids[b"<|end_of_text|>"]) == b"" and to.decode(t, ids[b"h"]) == b"h"
