"""Writes GGUF files for the tests (versions 2/3 layout: header, key/value pairs,
tensor descriptions, padding to 32, data).  Test-side only."""
from __future__ import annotations

import struct

import numpy as np

(U8, I8, U16, I16, U32, I32, F32, BOOL, STRING, ARRAY, U64, I64, F64) = range(13)
GGML_F32, GGML_F16 = 0, 1
_FMT = {U8: "<B", I8: "<b", U16: "<H", I16: "<h", U32: "<I", I32: "<i", F32: "<f", BOOL: "<B", U64: "<Q", I64: "<q",
        F64: "<d"}


def gstr(s) -> bytes:
    b = s if isinstance(s, bytes) else s.encode()
    return struct.pack("<Q", len(b)) + b


def value(ty: int, v) -> bytes:
    if ty == STRING:
        return gstr(v)
    if ty == ARRAY:
        elem, items = v
        return struct.pack("<IQ", elem, len(items)) + b"".join(value(elem, x) for x in items)
    return struct.pack(_FMT[ty], v)


def write_gguf(path, kv: list, tensors: list, version: int = 3) -> None:
    """kv: [(key, type, value)]; tensors: [(name, numpy array float32 | uint16 (binary16 bits), dims)].
    dims are written as given (GGUF lists the fastest-varying dimension first)."""
    head = struct.pack("<IIQQ", 0x46554747, version, len(tensors), len(kv))
    body = b"".join(gstr(k) + struct.pack("<I", ty) + value(ty, v) for k, ty, v in kv)
    infos, blobs, off = b"", [], 0
    for name, arr, dims in tensors:
        arr = np.ascontiguousarray(arr)
        ty = GGML_F32 if arr.dtype == np.float32 else GGML_F16
        assert arr.dtype in (np.float32, np.uint16) and int(np.prod(dims)) == arr.size
        infos += gstr(name) + struct.pack("<I", len(dims)) + struct.pack(f"<{len(dims)}Q", *dims) + struct.pack("<IQ", ty, off)
        blob = arr.tobytes()
        blob += b"\0" * (-len(blob) % 32)
        blobs.append(blob)
        off += len(blob)
    pre = head + body + infos
    pre += b"\0" * (-len(pre) % 32)
    with open(path, "wb") as f:
        f.write(pre + b"".join(blobs))


def llama_kv(shape, arch: str = "llama", with_kv_heads: bool = True, with_rope: bool = True, context=None,
             noise: bool = True) -> list:
    """The key/value pairs gguf_extract_config reads (loader.cpp:213-339), optionally with pairs of
    every other type in front of and between them, which a reader has to step over."""
    kv = []
    if noise:
        kv += [("general.name", STRING, "synthetic"), ("general.quantization_version", U32, 2),
               ("x.u8", U8, 7), ("x.i8", I8, -3), ("x.u16", U16, 65535), ("x.i16", I16, -2), ("x.i32", I32, -5),
               ("x.bool", BOOL, 1), ("x.u64", U64, 2 ** 40), ("x.i64", I64, -2 ** 40), ("x.f64", F64, 2.5),
               ("x.floats", ARRAY, (F32, [0.5, 1.5, 2.5])), ("x.nested", ARRAY, (ARRAY, [(U16, [1, 2]), (U16, [3])])),
               ("x.strings", ARRAY, (STRING, ["a", "bc", ""]))]
    kv += [("general.architecture", STRING, arch),
           (f"{arch}.embedding_length", U32, shape.dim), (f"{arch}.feed_forward_length", U32, shape.hidden_dim),
           (f"{arch}.block_count", U32, shape.n_layers), (f"{arch}.attention.head_count", U32, shape.n_heads)]
    if with_kv_heads:
        kv.append((f"{arch}.attention.head_count_kv", U32, shape.n_kv_heads))
    kv.append((f"{arch}.context_length", U32, context if context is not None else shape.seq_len))
    if with_rope:
        kv.append((f"{arch}.rope.freq_base", F32, float(shape.rope_base)))
    kv.append(("tokenizer.ggml.tokens", ARRAY, (STRING, [f"t{i}" for i in range(shape.vocab_size)])))
    if noise:
        kv.append(("tokenizer.ggml.scores", ARRAY, (F32, [0.0] * 4)))
    return kv


NAMES = {1: "attn_norm", 2: "attn_q", 3: "attn_k", 4: "attn_v", 5: "attn_output", 6: "ffn_norm", 7: "ffn_gate",
         8: "ffn_down", 9: "ffn_up"}


def llama_tensors(shape, weights: dict, f16_matrices: bool, f16_embedding: bool = False) -> list:
    """The tensors gguf_init_weights looks up (loader.cpp:446-541), split per layer.  weights: tensor id ->
    array in the stacked layout (matrices float32, or uint16 binary16 bits when f16_matrices)."""
    out = []
    emb = np.ascontiguousarray(weights[0], dtype=np.float32)
    if f16_embedding:
        emb = emb.astype(np.float16).view(np.uint16)
    out.append(("token_embd.weight", emb.reshape(-1), (shape.dim, shape.vocab_size)))
    for l in range(shape.n_layers):
        for t, nm in NAMES.items():
            a = np.ascontiguousarray(weights[t][l])
            dims = tuple(reversed(a.shape))
            out.append((f"blk.{l}.{nm}.weight", a.reshape(-1), dims))
    out.append(("output_norm.weight", np.ascontiguousarray(weights[10], dtype=np.float32), (shape.dim,)))
    if not shape.tied:
        out.append(("output.weight", np.ascontiguousarray(weights[11]).reshape(-1), (shape.dim, shape.vocab_size)))
    return out
