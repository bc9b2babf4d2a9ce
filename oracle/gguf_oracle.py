"""CPU restatement of the reference's GGUF reader (src/gguf.cpp and
src/loader.cpp:213-541) in numpy.

TEST INFRASTRUCTURE ONLY: the checker for lpp_gguf_* / lpp_model_load_gguf.  Only
the test-suite imports it; the product never does.

Pinning status:
  parse            the reference's own known sizes are none (its tests hold no GGUF
                   file); pinned by live equality with the compiled reference
                   (oracle/_ref: gguf_open + gguf_extract_config + gguf_init_weights)
                   on files written by tests/gguf_writer.py -- config fields and
                   every stacked weight array bit for bit, F32 and F16, tied and
                   untied, with key/value pairs of every type in front of the ones
                   that are read -- and by a hand-assembled byte string whose
                   offsets are worked out in the test
  extract_config   same runs (loader.cpp:213-339), incl. the defaults for a missing
                   head_count_kv / rope.freq_base and the 16384 cap
  stacked_weights  same runs (loader.cpp:423-541, CPU half)
"""
from __future__ import annotations

import struct

import numpy as np

MAGIC = 0x46554747  # gguf.h:8
(U8, I8, U16, I16, U32, I32, F32, BOOL, STRING, ARRAY, U64, I64, F64) = range(13)  # gguf.h:20-34
GGML_F32, GGML_F16 = 0, 1  # gguf.h:10-12
_FIXED = {U8: 1, I8: 1, BOOL: 1, U16: 2, I16: 2, U32: 4, I32: 4, F32: 4, U64: 8, I64: 8, F64: 8}


class GgufError(ValueError):
    pass


def _skip(buf: bytes, pos: int, ty: int) -> int:
    """gguf.cpp:49-88: position after a value of the given type."""
    if ty in _FIXED:
        return pos + _FIXED[ty]
    if ty == STRING:
        (n,) = struct.unpack_from("<Q", buf, pos)
        return pos + 8 + n
    if ty == ARRAY:
        elem, count = struct.unpack_from("<IQ", buf, pos)
        pos += 12
        for _ in range(count):
            pos = _skip(buf, pos, elem)
        return pos
    raise GgufError(f"unknown value type {ty}")


def _string(buf: bytes, pos: int):
    (n,) = struct.unpack_from("<Q", buf, pos)
    return buf[pos + 8:pos + 8 + n].decode("utf-8", "replace"), pos + 8 + n


def parse(buf: bytes) -> dict:
    """gguf_open, gguf.cpp:125-266.  Returns {'version', 'meta': {key: (type, value offset)},
    'tensors': {name: (type, dims, offset)}, 'data_start'}; first occurrence of a name wins, as
    the reference's linear searches do (gguf.cpp:91-98, 292-299)."""
    magic, version, n_tensors, n_meta = struct.unpack_from("<IIQQ", buf, 0)
    if magic != MAGIC:
        raise GgufError("magic")
    if version < 2 or version > 3:  # gguf.cpp:174-178
        raise GgufError("version")
    pos = 24
    meta, tensors = {}, {}
    for _ in range(n_meta):  # gguf.cpp:189-214
        key, pos = _string(buf, pos)
        (ty,) = struct.unpack_from("<I", buf, pos)
        pos += 4
        meta.setdefault(key, (ty, pos))
        pos = _skip(buf, pos, ty)
    for _ in range(n_tensors):  # gguf.cpp:218-255
        name, pos = _string(buf, pos)
        (nd,) = struct.unpack_from("<I", buf, pos)
        dims = struct.unpack_from(f"<{nd}Q", buf, pos + 4)
        ty, off = struct.unpack_from("<IQ", buf, pos + 4 + 8 * nd)
        pos += 4 + 8 * nd + 12
        tensors.setdefault(name, (ty, dims, off))
    data_start = (pos + 31) & ~31  # gguf.cpp:259-261
    if pos > len(buf):
        raise GgufError("truncated")
    return {"version": version, "meta": meta, "tensors": tensors, "data_start": data_start}


def _get(buf: bytes, g: dict, key: str, ty: int, fmt: str):
    """The typed getters of gguf.cpp:311-336: absent, or of another type, reads as missing."""
    e = g["meta"].get(key)
    if e is None or e[0] != ty:
        return None
    return struct.unpack_from(fmt, buf, e[1])[0]


def extract_config(buf: bytes, g: dict) -> dict:
    """gguf_extract_config (loader.cpp:213-339) + the precision test of gguf_init_weights (:426-433)."""
    e = g["meta"].get("general.architecture")
    if e is None or e[0] != STRING:
        raise GgufError("general.architecture")
    arch, _ = _string(buf, e[1])
    prefix = arch + "."
    cfg = {}
    for field, key in (("dim", "embedding_length"), ("hidden_dim", "feed_forward_length"), ("n_layers", "block_count"),
                       ("n_heads", "attention.head_count"), ("seq_len", "context_length")):
        v = _get(buf, g, prefix + key, U32, "<I")
        if v is None:
            raise GgufError(prefix + key)
        cfg[field] = v
    kv = _get(buf, g, prefix + "attention.head_count_kv", U32, "<I")
    cfg["n_kv_heads"] = kv if kv else cfg["n_heads"]  # :273-277 (0 treated as absent, as the product does)
    rope = _get(buf, g, prefix + "rope.freq_base", F32, "<f")
    cfg["rope_base"] = np.float32(10000.0 if rope is None else rope)  # :289-292
    e = g["meta"].get("tokenizer.ggml.tokens")  # :297-303
    count = 0
    if e is not None and e[0] == ARRAY:
        elem, count = struct.unpack_from("<IQ", buf, e[1])
        if elem != STRING:
            count = 0
    if count == 0:
        raise GgufError("tokenizer.ggml.tokens")
    cfg["vocab_size"] = count
    cfg["seq_len"] = min(cfg["seq_len"], 16384)  # :333-336
    q0 = g["tensors"].get("blk.0.attn_q.weight")
    cfg["fp16"] = q0 is not None and q0[0] == GGML_F16
    return cfg


def tensor(buf: bytes, g: dict, name: str):
    """gguf_tensor_data (gguf.cpp:301-303): (ggml type, flat array) -- float32 or binary16 bit patterns."""
    ty, dims, off = g["tensors"][name]
    n = int(np.prod(dims))
    dt = {GGML_F32: np.float32, GGML_F16: np.uint16}[ty]
    return ty, np.frombuffer(buf, dtype=dt, count=n, offset=g["data_start"] + off)


def _widen(ty: int, a: np.ndarray) -> np.ndarray:
    """copy_tensor_data (loader.cpp:381-401): F32 as is, F16 widened exactly."""
    return a.astype(np.float32) if ty == GGML_F32 else a.view(np.float16).astype(np.float32)


def stacked_weights(buf: bytes, g: dict, cfg: dict):
    """gguf_init_weights, CPU half (loader.cpp:423-541): the twelve fp32 arrays, per-layer tensors
    stacked, and whether the classifier is tied.  Order = transformerWeights (model.h:34-55)."""
    L = cfg["n_layers"]

    def one(name):
        return _widen(*tensor(buf, g, name))

    def per_layer(suffix):
        return np.concatenate([one(f"blk.{l}.{suffix}.weight") for l in range(L)])

    emb = one("token_embd.weight")
    tied = "output.weight" not in g["tensors"]
    out = [emb, per_layer("attn_norm"), per_layer("attn_q"), per_layer("attn_k"), per_layer("attn_v"),
           per_layer("attn_output"), per_layer("ffn_norm"), per_layer("ffn_gate"), per_layer("ffn_down"),
           per_layer("ffn_up"), one("output_norm.weight"), emb if tied else one("output.weight")]
    return out, tied
