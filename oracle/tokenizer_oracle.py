"""CPU restatement of the reference's tokenizer (src/tokenizer.cpp,
src/loader.cpp:648-699) in plain Python.

TEST INFRASTRUCTURE ONLY: the checker for lpp_tokenizer_*.  Only the test-suite
imports it; the product never does.

Pinning status (the reference's own tests hold no tokenizer case):
  load_file, from_gguf   live equality with the compiled reference (oracle/_ref:
                         load_tokenizer, gguf_init_tokenizer) on kind, size, scores
                         and, through decode, every string
  encode                 live equality with the compiled reference's encode on
                         texts chosen so that a wrong merge order, a missing blank
                         in front, a wrong marker, a lost byte fallback or a wrong
                         tie-break each change the ids; plus hand-worked cases
  decode                 live equality with decode_token over a whole vocabulary
                         (markers, byte tokens, other "<...>" entries, 255-byte cut)
"""
from __future__ import annotations

import re
import struct

SENTENCEPIECE, BPE = 0, 1  # TokenizerType, tokenizer.h:4-7


class Tok:
    def __init__(self, kind: int, vocab: list, scores: list, max_token_len: int):
        self.kind, self.vocab, self.scores, self.max_token_len = kind, vocab, scores, max_token_len
        self.ids = {}
        for i, s in enumerate(vocab):  # tokenizer.cpp:131-137: the last of equal strings wins
            self.ids[s] = i


def load_file(data: bytes, vocab_size: int) -> Tok:
    """load_tokenizer, tokenizer.cpp:15-55."""
    (max_len,) = struct.unpack_from("<i", data, 0)
    pos, vocab, scores = 4, [], []
    for _ in range(vocab_size):
        score, n = struct.unpack_from("<fi", data, pos)
        vocab.append(data[pos + 8:pos + 8 + n])
        scores.append(score)
        pos += 8 + n
    return Tok(SENTENCEPIECE, vocab, scores, max_len)


def from_gguf(model, tokens: list, scores) -> Tok:
    """gguf_init_tokenizer, loader.cpp:648-699: model = tokenizer.ggml.model or None."""
    kind = BPE if model == "gpt2" else SENTENCEPIECE
    if scores is None or len(scores) != len(tokens):
        scores = [0.0] * len(tokens)
    cstr = [t.split(b"\0")[0] for t in tokens]  # the reference holds C strings
    return Tok(kind, cstr, list(scores), max((len(t) for t in cstr), default=0))


def encode(t: Tok, text: bytes, max_tokens: int = 1 << 30) -> list:
    """encode, tokenizer.cpp:148-235."""
    cur = []
    if t.kind == BPE:
        bos = t.ids.get(b"<|begin_of_text|>", -1)
        if bos != -1:
            cur.append(bos)
    elif len(t.vocab) > 1 and t.vocab[1] == b"<s>":
        cur.append(1)
    marker = b"\xC4\xA0" if t.kind == BPE else b"\xE2\x96\x81"
    for ch in b" " + text:
        i = t.ids.get(marker if ch == 0x20 else bytes([ch]), -1)
        if i == -1:
            i = t.ids.get(b"<0x%02X>" % ch, -1)
        if i != -1:
            cur.append(i)
    while len(cur) >= 2:
        best_score, best_idx, best_tok = -1e10, -1, -1
        for i in range(len(cur) - 1):
            j = t.ids.get(t.vocab[cur[i]] + t.vocab[cur[i + 1]], -1)
            if j != -1 and t.scores[j] > best_score:
                best_score, best_idx, best_tok = t.scores[j], i, j
        if best_idx == -1:
            break
        cur[best_idx:best_idx + 2] = [best_tok]
    return cur[:max_tokens]


def decode(t: Tok, token_id: int) -> bytes:
    """decode_token, tokenizer.cpp:61-123 (as a C string: up to the first NUL)."""
    raw = t.vocab[token_id].split(b"\0")[0]
    if raw[:1] == b"<" and raw[-1:] == b">":
        # :72-79: six bytes, "<0x", then sscanf's %02X -- at most two characters, an optional sign
        # among them, at least one hexadecimal digit; what follows them is not looked at
        if len(raw) == 6 and raw[1:3] == b"0x":
            m = re.match(rb"([+-]?)([0-9A-Fa-f]+)", raw[3:5])
            if m:
                v = int(m.group(2), 16) * (-1 if m.group(1) == b"-" else 1)
                return bytes([v & 0xFF]).split(b"\0")[0]
        return b""
    out, i = bytearray(), 0
    while i < len(raw) and len(out) < 255:
        if t.kind == BPE and raw[i:i + 2] == b"\xC4\xA0":
            out.append(0x20)
            i += 2
        elif t.kind == BPE and raw[i:i + 2] == b"\xC4\x8A":
            out.append(0x0A)
            i += 2
        elif t.kind != BPE and raw[i:i + 3] == b"\xE2\x96\x81":
            out.append(0x20)
            i += 3
        else:
            out.append(raw[i])
            i += 1
    return bytes(out)
