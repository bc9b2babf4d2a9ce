"""Python handle on an lpp_model (section B of include/lpp.h) plus the seeded
synthetic-weight recipe shared by the tests and the benchmark.

Nothing here computes: every call forwards to liblpp_hip.so.
"""
from __future__ import annotations

import ctypes as C
from dataclasses import dataclass, asdict

import numpy as np

from . import capi


@dataclass(frozen=True)
class Shape:
    """Fields of Config (src/model.h:21-31) plus whether the classifier is tied."""
    dim: int
    hidden_dim: int
    n_layers: int
    n_heads: int
    n_kv_heads: int
    vocab_size: int
    seq_len: int
    rope_base: float = 10000.0
    fp16: bool = True
    tied: bool = True

    @property
    def head_size(self) -> int:
        return self.dim // self.n_heads

    @property
    def kv_dim(self) -> int:
        return self.dim * self.n_kv_heads // self.n_heads

    def tensor_shape(self, t: int) -> tuple:
        L, d, h, v, kv = self.n_layers, self.dim, self.hidden_dim, self.vocab_size, self.kv_dim
        return {
            capi.T_TOKEN_EMBEDDING: (v, d), capi.T_RMS_ATT: (L, d), capi.T_WQ: (L, d, d),
            capi.T_WK: (L, kv, d), capi.T_WV: (L, kv, d), capi.T_WO: (L, d, d), capi.T_RMS_FFN: (L, d),
            capi.T_W1: (L, h, d), capi.T_W2: (L, d, h), capi.T_W3: (L, h, d), capi.T_RMS_FINAL: (d,),
            capi.T_WCLS: (v, d),
        }[t]

    def matrix_params(self) -> int:
        L, d, h, v, kv = self.n_layers, self.dim, self.hidden_dim, self.vocab_size, self.kv_dim
        return L * (2 * d * d + 2 * kv * d + 3 * h * d) + v * d

    def bytes_per_token(self, pos: int) -> float:
        """Algorithmic HBM bytes of one decode step at position pos: every weight
        matrix once, norm gains, the embedding row, K and V of pos+1 positions read
        once per KV head (binary16), and the new K/V written."""
        w = 2 if self.fp16 else 4
        L, d, kv = self.n_layers, self.dim, self.kv_dim
        return (w * self.matrix_params() + 4 * (2 * L + 1) * d + 4 * d
                + 2 * 2 * kv * L * (pos + 1) + 2 * 2 * kv * L)


# The five benchmark shapes.
CONFIGS = {
    "c1_llama2c_15m_fp32": Shape(288, 768, 6, 6, 6, 32000, 256, 10000.0, fp16=False, tied=True),
    "c2_tinyllama_1b_fp16": Shape(2048, 5632, 22, 32, 4, 32000, 2048, 10000.0, fp16=True, tied=False),
    "c3_llama32_1b_fp16": Shape(2048, 8192, 16, 32, 8, 128256, 2048, 500000.0, fp16=True, tied=True),
    "c4_llama32_1b_longctx_fp16": Shape(2048, 8192, 16, 32, 8, 128256, 16384, 500000.0, fp16=True, tied=True),
    "c5_llama3_8b_fp16": Shape(4096, 14336, 32, 32, 8, 128256, 2048, 500000.0, fp16=True, tied=False),
}

MATRIX_TENSORS = (capi.T_WQ, capi.T_WK, capi.T_WV, capi.T_WO, capi.T_W1, capi.T_W2, capi.T_W3, capi.T_WCLS)
GAIN_TENSORS = (capi.T_RMS_ATT, capi.T_RMS_FFN, capi.T_RMS_FINAL)


def synth_tensor(shape: Shape, t: int, seed: int) -> np.ndarray:
    """Host copy of one synthetic tensor: matrices and the embedding ~ N(0, 0.02)
    from stream (seed, tensor id); norm gains are 1.  For fp16 models matrices come
    back as binary16 bit patterns (uint16) and the embedding as those same
    binary16 values widened to fp32, which is what a GGUF F16 file gives the
    reference (src/loader.cpp:391-395)."""
    dims = shape.tensor_shape(t)
    n = int(np.prod(dims))
    stream = seed * 64 + t
    if t in GAIN_TENSORS:
        return np.ones(dims, dtype=np.float32)
    if t == capi.T_TOKEN_EMBEDDING:
        if shape.fp16:
            return capi.f16_to_f32(capi.synth_normal_f16(n, stream, 0.02)).reshape(dims)
        return capi.synth_normal_f32(n, stream, 0.02).reshape(dims)
    if t == capi.T_WCLS and shape.tied:
        emb = synth_tensor(shape, capi.T_TOKEN_EMBEDDING, seed)
        return capi.f32_to_f16(emb).reshape(dims) if shape.fp16 else emb
    if shape.fp16:
        return capi.synth_normal_f16(n, stream, 0.02).reshape(dims)
    return capi.synth_normal_f32(n, stream, 0.02).reshape(dims)


def write_checkpoint(path, shape: Shape, tensors: dict) -> None:
    """Writes a llama2.c checkpoint as the reference reads it (src/loader.cpp:134-172,
    18-66): seven ints, then the eleven fp32 tensors back to back, classifier tied."""
    assert not shape.fp16 and shape.tied, "the format holds fp32 tensors and a tied classifier"
    with open(path, "wb") as f:
        f.write(np.array([shape.dim, shape.hidden_dim, shape.n_layers, shape.n_heads, shape.n_kv_heads,
                          shape.vocab_size, shape.seq_len], dtype=np.int32).tobytes())
        for t in range(capi.T_WCLS):
            a = np.ascontiguousarray(tensors[t], dtype=np.float32)
            assert a.shape == shape.tensor_shape(t), (t, a.shape)
            f.write(a.tobytes())


class Checkpoint:
    """A llama2.c checkpoint mapped by lpp_checkpoint_open (host code, no GPU)."""

    def __init__(self, path):
        self.lib = capi.load()
        h = C.c_void_p()
        capi.check(self.lib.lpp_checkpoint_open(C.byref(h), str(path).encode()))
        self.handle = h
        cfg = capi.LppConfig()
        capi.check(self.lib.lpp_checkpoint_config(self.handle, C.byref(cfg)))
        self.config = cfg
        self.shape = Shape(cfg.dim, cfg.hidden_dim, cfg.n_layers, cfg.n_heads, cfg.n_kv_heads, cfg.vocab_size,
                           cfg.seq_len, cfg.rope_base, fp16=cfg.weight_precision == capi.WEIGHT_FP16, tied=True)

    def tensor(self, t: int) -> np.ndarray:
        """Copy of the named tensor, shaped."""
        p, n = C.c_void_p(), C.c_size_t()
        capi.check(self.lib.lpp_checkpoint_tensor(self.handle, t, C.byref(p), C.byref(n)))
        flat = np.ctypeslib.as_array(C.cast(p, C.POINTER(C.c_float)), shape=(n.value,))
        return flat.reshape(self.shape.tensor_shape(t)).copy()

    def tensor_offset(self, t: int) -> int:
        """Floats between the first weight of the file and the named tensor."""
        p, n, p0 = C.c_void_p(), C.c_size_t(), C.c_void_p()
        capi.check(self.lib.lpp_checkpoint_tensor(self.handle, t, C.byref(p), C.byref(n)))
        capi.check(self.lib.lpp_checkpoint_tensor(self.handle, capi.T_TOKEN_EMBEDDING, C.byref(p0), C.byref(n)))
        return (p.value - p0.value) // 4

    def close(self) -> None:
        if self.handle:
            self.lib.lpp_checkpoint_close(self.handle)
            self.handle = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


class Tokenizer:
    """lpp_tokenizer: the tokenizer of src/tokenizer.cpp (host code, no GPU)."""

    def __init__(self, handle):
        self.lib = capi.load()
        self.handle = handle
        n, kind, mx = C.c_int(), C.c_int(), C.c_int()
        capi.check(self.lib.lpp_tokenizer_info(handle, C.byref(n), C.byref(kind), C.byref(mx)))
        self.vocab_size, self.kind, self.max_token_len = n.value, kind.value, mx.value

    @classmethod
    def load(cls, path, vocab_size: int) -> "Tokenizer":
        h = C.c_void_p()
        capi.check(capi.load().lpp_tokenizer_load(C.byref(h), str(path).encode(), vocab_size))
        return cls(h)

    @classmethod
    def from_gguf(cls, g: "Gguf") -> "Tokenizer":
        h = C.c_void_p()
        capi.check(g.lib.lpp_tokenizer_from_gguf(C.byref(h), g.handle))
        return cls(h)

    def encode(self, text, max_tokens: int = 2048) -> list:
        raw = text if isinstance(text, bytes) else text.encode()
        out = np.empty(max(max_tokens, 1), dtype=np.int32)
        n = C.c_int()
        capi.check(self.lib.lpp_tokenizer_encode(self.handle, raw, C.c_void_p(out.ctypes.data), max_tokens, C.byref(n)))
        return out[:n.value].tolist()

    def decode(self, token_id: int) -> bytes:
        buf = C.create_string_buffer(256)
        capi.check(self.lib.lpp_tokenizer_decode(self.handle, token_id, buf, 256))
        return buf.value

    def close(self) -> None:
        if self.handle:
            self.lib.lpp_tokenizer_free(self.handle)
            self.handle = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


class Gguf:
    """A GGUF file mapped by lpp_gguf_open (host code, no GPU)."""

    def __init__(self, path):
        self.lib = capi.load()
        h = C.c_void_p()
        capi.check(self.lib.lpp_gguf_open(C.byref(h), str(path).encode()))
        self.handle = h

    @property
    def config(self) -> "capi.LppConfig":
        cfg = capi.LppConfig()
        capi.check(self.lib.lpp_gguf_config(self.handle, C.byref(cfg)))
        return cfg

    def shape(self, tied: bool) -> Shape:
        c = self.config
        return Shape(c.dim, c.hidden_dim, c.n_layers, c.n_heads, c.n_kv_heads, c.vocab_size, c.seq_len, c.rope_base,
                     fp16=c.weight_precision == capi.WEIGHT_FP16, tied=tied)

    def tensor(self, name: str) -> np.ndarray:
        """Copy of a named tensor, flat: float32, or binary16 bit patterns (uint16)."""
        p, ty, n = C.c_void_p(), C.c_int(), C.c_size_t()
        capi.check(self.lib.lpp_gguf_tensor(self.handle, name.encode(), C.byref(p), C.byref(ty), C.byref(n)))
        ctype, dtype = {capi.GGML_F32: (C.c_float, np.float32), capi.GGML_F16: (C.c_uint16, np.uint16)}[ty.value]
        return np.ctypeslib.as_array(C.cast(p, C.POINTER(ctype)), shape=(n.value,)).astype(dtype, copy=True)

    def has_tensor(self, name: str) -> bool:
        p, ty, n = C.c_void_p(), C.c_int(), C.c_size_t()
        return self.lib.lpp_gguf_tensor(self.handle, name.encode(), C.byref(p), C.byref(ty), C.byref(n)) == capi.LPP_OK

    def close(self) -> None:
        if self.handle:
            self.lib.lpp_gguf_close(self.handle)
            self.handle = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


class Model:
    def __init__(self, shape: Shape, _handle=None):
        self.shape = shape
        lib = capi.load()
        if _handle is not None:
            self.handle, self.lib = _handle, lib
            return
        cfg = capi.LppConfig(shape.dim, shape.hidden_dim, shape.n_layers, shape.n_heads, shape.n_kv_heads,
                             shape.vocab_size, shape.seq_len, shape.rope_base,
                             capi.WEIGHT_FP16 if shape.fp16 else capi.WEIGHT_FP32)
        h = C.c_void_p()
        capi.check(lib.lpp_model_create(C.byref(h), C.byref(cfg)))
        self.handle = h
        self.lib = lib

    @classmethod
    def from_checkpoint(cls, ck: "Checkpoint") -> "Model":
        """lpp_model_load_checkpoint: create, upload every tensor, tie the classifier."""
        h = C.c_void_p()
        capi.check(ck.lib.lpp_model_load_checkpoint(C.byref(h), ck.handle))
        return cls(ck.shape, _handle=h)

    @classmethod
    def from_gguf(cls, g: "Gguf") -> "Model":
        """lpp_model_load_gguf: create, gather the named tensors into the stacked layout, upload."""
        h = C.c_void_p()
        capi.check(g.lib.lpp_model_load_gguf(C.byref(h), g.handle))
        return cls(g.shape(tied=not g.has_tensor("output.weight")), _handle=h)

    def close(self) -> None:
        if self.handle:
            self.lib.lpp_model_destroy(self.handle)
            self.handle = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    # ---- weights ----
    def upload(self, t: int, host: np.ndarray, byte_offset: int = 0) -> None:
        host = np.ascontiguousarray(host)
        capi.check(self.lib.lpp_model_upload(self.handle, t, byte_offset, C.c_void_p(host.ctypes.data), host.nbytes))

    def tie_classifier(self) -> None:
        capi.check(self.lib.lpp_model_tie_classifier(self.handle))

    def load_synthetic(self, seed: int, keep: bool = False) -> dict:
        """Fill every tensor from the seeded recipe.  keep=True also returns the host
        arrays (for a CPU checker); otherwise each is dropped after upload."""
        kept = {}
        for t in range(12):
            if t == capi.T_WCLS and self.shape.tied:
                continue
            a = synth_tensor(self.shape, t, seed)
            self.upload(t, a)
            if keep:
                kept[t] = a
        if self.shape.tied:
            self.tie_classifier()
            if keep:
                emb = kept[capi.T_TOKEN_EMBEDDING]
                kept[capi.T_WCLS] = capi.f32_to_f16(emb).reshape(emb.shape) if self.shape.fp16 else emb
        return kept

    # ---- run ----
    def set_path(self, path: int) -> None:
        capi.check(self.lib.lpp_model_set_path(self.handle, path))

    def reset(self) -> None:
        capi.check(self.lib.lpp_model_reset(self.handle))

    def forward(self, token: int, pos: int, temperature: float = 0.0, topp: float = 1.0, penalty: float = 1.0,
                history=None, r: float = 0.0) -> int:
        out = C.c_int(-1)
        if history is not None and len(history) > 0:
            h = np.ascontiguousarray(history, dtype=np.int32)
            hp, hl = C.c_void_p(h.ctypes.data), int(h.size)
        else:
            hp, hl = None, 0
        capi.check(self.lib.lpp_forward(self.handle, token, pos, temperature, topp, penalty, hp, hl, r,
                                        C.byref(out)))
        return out.value

    def generate(self, first_token: int, start_pos: int, n_steps: int, temperature: float = 0.0,
                 topp: float = 1.0, penalty: float = 1.0, history=None, history_cap: int = 0, uniforms=None):
        """Returns (tokens[n_steps], history list after the run, LppGenStats)."""
        out = np.empty(n_steps, dtype=np.int32)
        hist = np.zeros(max(history_cap, 1), dtype=np.int32)
        hlen = C.c_int(0)
        if history is not None and len(history) > 0:
            hist[:len(history)] = history
            hlen.value = len(history)
        up = None
        if uniforms is not None:
            u = np.ascontiguousarray(uniforms, dtype=np.float32)
            assert u.size >= n_steps
            up = C.c_void_p(u.ctypes.data)
        stats = capi.LppGenStats()
        capi.check(self.lib.lpp_generate(self.handle, first_token, start_pos, n_steps, temperature, topp, penalty,
                                         C.c_void_p(hist.ctypes.data), C.byref(hlen), history_cap, up,
                                         C.c_void_p(out.ctypes.data), C.byref(stats)))
        return out, hist[:hlen.value].tolist(), stats

    def prefill_supported(self) -> bool:
        """Whether lpp_prefill (batched prefill on the matrix cores) takes this model."""
        return self.lib.lpp_prefill_supported(self.handle) == capi.LPP_OK

    def set_prefill_mode(self, mode: int) -> None:
        """capi.PREFILL_EXACT (binary16 head + remainder of the activations) or capi.PREFILL_FAST (head alone)."""
        capi.check(self.lib.lpp_model_set_prefill_mode(self.handle, mode))

    def prefill(self, tokens, start_pos: int = 0) -> None:
        """lpp_prefill: the KV cache entries of `tokens` at positions start_pos.., all layers, in one batch."""
        t = np.ascontiguousarray(tokens, dtype=np.int32)
        capi.check(self.lib.lpp_prefill(self.handle, C.c_void_p(t.ctypes.data), int(t.size), int(start_pos)))

    def run(self, prompt, steps: int, temperature: float = 0.0, topp: float = 1.0, uniforms=None,
            batched_prefill: bool = False):
        """lpp_run, the driver loop of src/main.cpp:139-232 (lpp_run_batched_prefill: the prompt in one batch).
        Returns (generated ids, LppRunResult)."""
        out = np.empty(max(steps, 1), dtype=np.int32)
        pp, pn = None, 0
        if prompt is not None and len(prompt) > 0:
            pr = np.ascontiguousarray(prompt, dtype=np.int32)
            pp, pn = C.c_void_p(pr.ctypes.data), int(pr.size)
        up = None
        if uniforms is not None:
            u = np.ascontiguousarray(uniforms, dtype=np.float32)
            need = max(steps, pn - 1)  # one draw per position: the prompt is prefilled to its end whatever `steps` is
            if u.size < need:
                raise ValueError(f"run: {u.size} uniforms for {need} positions (max(steps, len(prompt) - 1))")
            up = C.c_void_p(u.ctypes.data)
        res = capi.LppRunResult()
        entry = self.lib.lpp_run_batched_prefill if batched_prefill else self.lib.lpp_run
        capi.check(entry(self.handle, pp, pn, steps, temperature, topp, up, C.c_void_p(out.ctypes.data),
                         int(out.size), C.byref(res)))
        return out[:res.n_tokens].copy(), res

    def profile_kernels(self, pos: int, reps: int = 20) -> list:
        """[(name, launches_per_token, avg_ms, bytes_per_launch)] of the model's current path: the fused kernels, the
        persistent kernel, or (operator path) each operator of lpp.h section A as a stand-alone launch."""
        arr = (capi.LppKernelTime * 32)()
        n = C.c_int(0)
        capi.check(self.lib.lpp_profile_kernels(self.handle, pos, reps, arr, 32, C.byref(n)))
        return [(arr[i].name.decode(), arr[i].launches_per_token, arr[i].avg_ms, arr[i].bytes_per_launch)
                for i in range(n.value)]

    # ---- inspection ----
    def buffer(self, b: int, dtype=None) -> np.ndarray:
        p, n = C.c_void_p(), C.c_size_t()
        capi.check(self.lib.lpp_model_buffer_ptr(self.handle, b, C.byref(p), C.byref(n)))
        if dtype is None:
            dtype = np.uint16 if b in (capi.B_KEY_CACHE, capi.B_VALUE_CACHE) else np.float32
        out = np.empty(n.value // np.dtype(dtype).itemsize, dtype=dtype)
        capi.synchronize()
        capi.check(self.lib.lpp_memcpy_d2h(C.c_void_p(out.ctypes.data), p, n.value))
        return out

    def write_buffer(self, b: int, host: np.ndarray, byte_offset: int = 0) -> None:
        p, n = C.c_void_p(), C.c_size_t()
        capi.check(self.lib.lpp_model_buffer_ptr(self.handle, b, C.byref(p), C.byref(n)))
        host = np.ascontiguousarray(host)
        assert byte_offset + host.nbytes <= n.value
        capi.check(self.lib.lpp_memcpy_h2d(C.c_void_p(p.value + byte_offset), C.c_void_p(host.ctypes.data),
                                           host.nbytes))

    def buffer_ptr(self, b: int) -> int:
        p, n = C.c_void_p(), C.c_size_t()
        capi.check(self.lib.lpp_model_buffer_ptr(self.handle, b, C.byref(p), C.byref(n)))
        return p.value

    def tensor_ptr(self, t: int) -> int:
        p = C.c_void_p()
        capi.check(self.lib.lpp_model_tensor_ptr(self.handle, t, C.byref(p)))
        return p.value
