"""ctypes view of the CPU oracle (oracle/liblpp_oracle.so) and, where it was
built, of the compiled reference (oracle/_ref/liblpp_ref.so).  Test-side only."""
from __future__ import annotations

import ctypes as C
import subprocess
from pathlib import Path

import numpy as np

ROOT = Path(__file__).resolve().parent.parent
ORACLE_DIR = ROOT / "oracle"
ORACLE_SO = ORACLE_DIR / "liblpp_oracle.so"
REF_SO = ORACLE_DIR / "_ref" / "liblpp_ref.so"

_f32p = np.ctypeslib.ndpointer(dtype=np.float32, flags="C_CONTIGUOUS")
_i32p = np.ctypeslib.ndpointer(dtype=np.int32, flags="C_CONTIGUOUS")
_u16p = np.ctypeslib.ndpointer(dtype=np.uint16, flags="C_CONTIGUOUS")


class OrcConfig(C.Structure):
    _fields_ = [("dim", C.c_int), ("hidden_dim", C.c_int), ("n_layers", C.c_int), ("n_heads", C.c_int),
                ("n_kv_heads", C.c_int), ("vocab_size", C.c_int), ("seq_len", C.c_int), ("rope_base", C.c_float)]


class OrcWeights(C.Structure):
    _fields_ = [(n, C.c_void_p) for n in
                ("token_embedding_table", "rms_att_weight", "wq", "wk", "wv", "wo", "rms_ffn_weight", "w1", "w2",
                 "w3", "rms_final_weight", "w_cls")] + [("w_is_f16", C.c_int)]


class OrcState(C.Structure):
    _fields_ = [(n, C.POINTER(C.c_float)) for n in
                ("x", "xb", "xb2", "hb", "he", "q", "k", "v", "att", "logits", "key_cache", "value_cache")] + \
               [("kv_round_f16", C.c_int)]


class OrcRunResult(C.Structure):
    _fields_ = [("n_tokens", C.c_int), ("final_pos", C.c_int), ("stopped_by_eos", C.c_int),
                ("reported_count", C.c_int), ("history_len", C.c_int), ("history", C.c_int * 64)]


REF_EXE = ORACLE_DIR / "_ref" / "lighterpp_ref"

_oracle = None
_ref = None


def build_oracle() -> None:
    subprocess.run(["make", "-C", str(ORACLE_DIR), "liblpp_oracle.so"], check=True, capture_output=True)


def oracle() -> C.CDLL:
    global _oracle
    if _oracle is not None:
        return _oracle
    if not ORACLE_SO.exists():
        build_oracle()
    lib = C.CDLL(str(ORACLE_SO))
    lib.orc_naive_matmul.argtypes = [_f32p, _f32p, _f32p, C.c_int, C.c_int]
    lib.orc_matmul_f16w.argtypes = [_f32p, _f32p, _u16p, C.c_int, C.c_int]
    lib.orc_rmsnorm.argtypes = [_f32p, _f32p, _f32p, C.c_int]
    lib.orc_rope.argtypes = [_f32p, _f32p, C.c_int, C.c_int, C.c_int, C.c_int, C.c_float]
    lib.orc_softmax.argtypes = [_f32p, C.c_int]
    lib.orc_swiglu.argtypes = [_f32p, _f32p, _f32p, C.c_int]
    lib.orc_f16_to_f32.argtypes = [C.c_uint16]
    lib.orc_f16_to_f32.restype = C.c_float
    lib.orc_f32_to_f16_rn.argtypes = [C.c_float]
    lib.orc_f32_to_f16_rn.restype = C.c_uint16
    lib.orc_state_alloc.argtypes = [C.POINTER(OrcState), C.POINTER(OrcConfig)]
    lib.orc_state_free.argtypes = [C.POINTER(OrcState)]
    lib.orc_attention.argtypes = [C.POINTER(OrcState), C.POINTER(OrcWeights), C.POINTER(OrcConfig), C.c_int, C.c_int]
    lib.orc_transformer_block.argtypes = lib.orc_attention.argtypes
    lib.orc_forward_logits.argtypes = [C.c_int, C.c_int, C.POINTER(OrcState), C.POINTER(OrcWeights),
                                       C.POINTER(OrcConfig)]
    lib.orc_sample.argtypes = [_f32p, C.c_int, C.c_float, C.c_float, C.c_float, C.c_void_p, C.c_int, C.c_float]
    lib.orc_sample.restype = C.c_int
    lib.orc_sample_cdf.argtypes = [_f32p, C.c_int, C.c_float, C.c_float, C.c_void_p, C.c_int, C.c_float,
                                   C.POINTER(C.c_float), C.POINTER(C.c_float)]
    lib.orc_sample_cdf.restype = C.c_int
    lib.orc_forward.argtypes = [C.c_int, C.c_int, C.POINTER(OrcState), C.POINTER(OrcWeights), C.POINTER(OrcConfig),
                                C.c_float, C.c_float, C.c_float, C.c_void_p, C.c_int, C.c_float]
    lib.orc_forward.restype = C.c_int
    lib.orc_history_push.argtypes = [_i32p, C.POINTER(C.c_int), C.c_int, C.c_int]
    lib.orc_run.argtypes = [C.c_void_p, C.c_int, C.c_int, C.c_float, C.c_float, C.c_void_p, C.POINTER(OrcState),
                            C.POINTER(OrcWeights), C.POINTER(OrcConfig), C.c_void_p, C.c_int, C.POINTER(OrcRunResult)]
    lib.orc_run.restype = C.c_int
    lib.orc_checkpoint_parse.argtypes = [C.c_void_p, C.c_size_t, C.POINTER(OrcConfig), C.POINTER(C.c_size_t),
                                         C.POINTER(C.c_size_t)]
    lib.orc_checkpoint_parse.restype = C.c_int
    _oracle = lib
    return lib


def have_ref() -> bool:
    return REF_SO.exists()


def ref() -> C.CDLL:
    global _ref
    if _ref is not None:
        return _ref
    lib = C.CDLL(str(REF_SO))
    lib.ref_naive_matmul.argtypes = [_f32p, _f32p, _f32p, C.c_int, C.c_int]
    lib.ref_rmsnorm.argtypes = [_f32p, _f32p, _f32p, C.c_int]
    lib.ref_rope.argtypes = [_f32p, _f32p, C.c_int, C.c_int, C.c_int, C.c_int, C.c_float]
    lib.ref_softmax.argtypes = [_f32p, C.c_int]
    lib.ref_swiglu.argtypes = [_f32p, _f32p, _f32p, C.c_int]
    lib.ref_srand.argtypes = [C.c_uint]
    lib.ref_next_uniform.restype = C.c_float
    lib.ref_sample.argtypes = [_f32p, C.c_int, C.c_float, C.c_float, C.c_float, C.c_void_p, C.c_int]
    lib.ref_sample.restype = C.c_int
    lib.ref_model_create.argtypes = [C.c_int] * 7 + [C.c_float] + [C.c_void_p] * 12
    lib.ref_model_create.restype = C.c_void_p
    lib.ref_model_destroy.argtypes = [C.c_void_p]
    lib.ref_forward.argtypes = [C.c_void_p, C.c_int, C.c_int, C.c_float, C.c_float, C.c_float, C.c_void_p, C.c_int]
    lib.ref_forward.restype = C.c_int
    lib.ref_attention.argtypes = [C.c_void_p, C.c_int, C.c_int]
    lib.ref_transformer_block.argtypes = [C.c_void_p, C.c_int, C.c_int]
    lib.ref_state_buffer.argtypes = [C.c_void_p, C.c_int]
    lib.ref_state_buffer.restype = C.POINTER(C.c_float)
    lib.ref_checkpoint_layout.argtypes = [C.c_char_p, C.POINTER(C.c_int), C.POINTER(C.c_float),
                                          C.POINTER(C.c_longlong)]
    lib.ref_checkpoint_layout.restype = C.c_int
    lib.ref_gguf_load.argtypes = [C.c_char_p, C.POINTER(C.c_int), C.POINTER(C.POINTER(C.c_float))]
    lib.ref_gguf_load.restype = C.c_void_p
    lib.ref_gguf_free.argtypes = [C.c_void_p]
    _ref = lib
    return lib


WEIGHT_FIELDS = ["token_embedding_table", "rms_att_weight", "wq", "wk", "wv", "wo", "rms_ffn_weight", "w1", "w2",
                 "w3", "rms_final_weight", "w_cls"]
STATE_FIELDS = ["x", "xb", "xb2", "hb", "he", "q", "k", "v", "att", "logits", "key_cache", "value_cache"]


class OracleModel:
    """The oracle's forward() over host weight arrays.

    weights: dict tensor-id (0..11, the order of WEIGHT_FIELDS) -> numpy array;
    matrices are float32, or uint16 binary16 bit patterns when fp16=True."""

    def __init__(self, shape, weights: dict, fp16: bool, kv_round_f16: bool = False):
        self.lib = oracle()
        self.shape = shape
        self.cfg = OrcConfig(shape.dim, shape.hidden_dim, shape.n_layers, shape.n_heads, shape.n_kv_heads,
                             shape.vocab_size, shape.seq_len, shape.rope_base)
        self._keep = {t: np.ascontiguousarray(a) for t, a in weights.items()}
        self.w = OrcWeights()
        for t, name in enumerate(WEIGHT_FIELDS):
            setattr(self.w, name, self._keep[t].ctypes.data)
        self.w.w_is_f16 = 1 if fp16 else 0
        self.s = OrcState()
        if self.lib.orc_state_alloc(C.byref(self.s), C.byref(self.cfg)) != 0:
            raise MemoryError("orc_state_alloc failed")
        self.s.kv_round_f16 = 1 if kv_round_f16 else 0

    def close(self):
        if self.s.x:
            self.lib.orc_state_free(C.byref(self.s))

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def sizes(self):
        p = self.shape
        kv_dim = p.dim * p.n_kv_heads // p.n_heads
        cache = p.n_layers * p.seq_len * kv_dim
        return {"x": p.dim, "xb": p.dim, "xb2": p.dim, "hb": p.hidden_dim, "he": p.hidden_dim, "q": p.dim,
                "k": kv_dim, "v": kv_dim, "att": p.n_heads * p.seq_len, "logits": p.vocab_size,
                "key_cache": cache, "value_cache": cache}

    def buf(self, name: str) -> np.ndarray:
        """Live numpy view of a state buffer."""
        n = self.sizes()[name]
        return np.ctypeslib.as_array(getattr(self.s, name), shape=(n,))

    def forward_logits(self, token: int, pos: int) -> np.ndarray:
        self.lib.orc_forward_logits(token, pos, C.byref(self.s), C.byref(self.w), C.byref(self.cfg))
        return self.buf("logits").copy()

    def transformer_block(self, layer: int, pos: int):
        self.lib.orc_transformer_block(C.byref(self.s), C.byref(self.w), C.byref(self.cfg), layer, pos)

    def attention(self, layer: int, pos: int):
        self.lib.orc_attention(C.byref(self.s), C.byref(self.w), C.byref(self.cfg), layer, pos)

    def forward(self, token, pos, temperature=0.0, topp=1.0, penalty=1.0, history=None, r=0.0) -> int:
        if history is not None and len(history) > 0:
            h = np.ascontiguousarray(history, dtype=np.int32)
            hp, hl = h.ctypes.data, int(h.size)
        else:
            hp, hl = None, 0
        return self.lib.orc_forward(token, pos, C.byref(self.s), C.byref(self.w), C.byref(self.cfg), temperature,
                                    topp, penalty, hp, hl, r)


    def run(self, prompt, steps: int, temperature: float = 0.0, topp: float = 1.0, uniforms=None):
        """orc_run, the driver loop of main.cpp:139-232.  Returns (generated ids, OrcRunResult)."""
        out = np.empty(max(steps, 1), dtype=np.int32)
        pp, pn = None, 0
        if prompt is not None and len(prompt) > 0:
            pr = np.ascontiguousarray(prompt, dtype=np.int32)
            pp, pn = pr.ctypes.data, int(pr.size)
        up = None
        if uniforms is not None:
            u = np.ascontiguousarray(uniforms, dtype=np.float32)
            up = u.ctypes.data
        res = OrcRunResult()
        rc = self.lib.orc_run(pp, pn, steps, temperature, topp, up, C.byref(self.s), C.byref(self.w),
                              C.byref(self.cfg), out.ctypes.data, int(out.size), C.byref(res))
        assert rc == 0
        return out[:res.n_tokens].copy(), res


def orc_checkpoint_parse(data: bytes):
    """(status, OrcConfig, offsets[12], counts[12]) of a llama2.c checkpoint held in memory."""
    cfg = OrcConfig()
    off = (C.c_size_t * 12)()
    cnt = (C.c_size_t * 12)()
    buf = C.create_string_buffer(data, len(data))
    rc = oracle().orc_checkpoint_parse(buf, len(data), C.byref(cfg), off, cnt)
    return rc, cfg, list(off), list(cnt)


def ref_checkpoint_layout(path):
    """(header[7], rope_base, offsets[12]) as the compiled reference reads the file."""
    hdr = (C.c_int * 7)()
    rb = C.c_float()
    off = (C.c_longlong * 12)()
    rc = ref().ref_checkpoint_layout(str(path).encode(), hdr, C.byref(rb), off)
    assert rc == 0
    return list(hdr), rb.value, list(off)


def fresh_ref(tmp_dir) -> C.CDLL:
    """A private copy of the compiled reference, with its own file-scope statics (the
    tokenizer keeps its string-to-id map in one, built from the first vocabulary it sees)."""
    import shutil
    import uuid
    dst = Path(tmp_dir) / f"liblpp_ref_{uuid.uuid4().hex}.so"
    shutil.copy(REF_SO, dst)
    lib = C.CDLL(str(dst))
    lib.ref_tokenizer_load.argtypes = [C.c_char_p, C.c_int]
    lib.ref_tokenizer_load.restype = C.c_void_p
    lib.ref_tokenizer_from_gguf.argtypes = [C.c_char_p]
    lib.ref_tokenizer_from_gguf.restype = C.c_void_p
    for f in ("ref_tokenizer_kind", "ref_tokenizer_vocab_size", "ref_tokenizer_max_token_len"):
        getattr(lib, f).argtypes = [C.c_void_p]
    lib.ref_tokenizer_score.argtypes = [C.c_void_p, C.c_int]
    lib.ref_tokenizer_score.restype = C.c_float
    lib.ref_encode.argtypes = [C.c_void_p, C.c_char_p, C.c_void_p, C.c_int]
    lib.ref_decode.argtypes = [C.c_void_p, C.c_int]
    lib.ref_decode.restype = C.c_char_p
    return lib


def ref_encode(lib, handle, text: bytes, max_tokens: int = 4096) -> list:
    out = np.empty(max_tokens, dtype=np.int32)
    n = lib.ref_encode(handle, text, out.ctypes.data, max_tokens)
    return out[:n].tolist()


def ref_gguf_load(path):
    """The compiled reference's reading of a GGUF file: (config dict, [12 fp32 arrays]) or None
    when it refuses the file.  Arrays are copies."""
    cfg = (C.c_int * 9)()
    ptrs = (C.POINTER(C.c_float) * 12)()
    h = ref().ref_gguf_load(str(path).encode(), cfg, ptrs)
    if not h:
        return None
    c = dict(zip(["dim", "hidden_dim", "n_layers", "n_heads", "n_kv_heads", "vocab_size", "seq_len"], list(cfg)[:7]))
    c["rope_base"] = np.array([cfg[7]], dtype=np.int32).view(np.float32)[0]
    c["fp16"] = cfg[8] == 1
    kv = c["dim"] // c["n_heads"] * c["n_kv_heads"]
    L, d, hd, v = c["n_layers"], c["dim"], c["hidden_dim"], c["vocab_size"]
    counts = [v * d, L * d, L * d * d, L * kv * d, L * kv * d, L * d * d, L * d, L * hd * d, L * d * hd, L * hd * d, d, v * d]
    arrays = [np.ctypeslib.as_array(ptrs[i], shape=(counts[i],)).copy() for i in range(12)]
    tied = C.addressof(ptrs[11].contents) == C.addressof(ptrs[0].contents)
    ref().ref_gguf_free(h)
    return c, arrays, tied


def orc_sample(logits: np.ndarray, temperature, topp, penalty, history, r) -> tuple:
    """Runs the oracle sampler on a copy; returns (token, mutated logits)."""
    lg = np.ascontiguousarray(logits, dtype=np.float32).copy()
    if history is not None and len(history) > 0:
        h = np.ascontiguousarray(history, dtype=np.int32)
        hp, hl = h.ctypes.data, int(h.size)
    else:
        hp, hl = None, 0
    tok = oracle().orc_sample(lg, lg.size, temperature, topp, penalty, hp, hl, r)
    return tok, lg


def orc_sample_cdf(logits: np.ndarray, temperature, penalty, history, r) -> tuple:
    """(token, cdf just below the token's bucket, cdf at its upper edge)."""
    lg = np.ascontiguousarray(logits, dtype=np.float32).copy()
    if history is not None and len(history) > 0:
        h = np.ascontiguousarray(history, dtype=np.int32)
        hp, hl = h.ctypes.data, int(h.size)
    else:
        hp, hl = None, 0
    lo, hi = C.c_float(), C.c_float()
    tok = oracle().orc_sample_cdf(lg, lg.size, temperature, penalty, hp, hl, r, C.byref(lo), C.byref(hi))
    return tok, lo.value, hi.value


class RefModel:
    """forward() of the compiled reference over fp32 host weights (tensor ids as above)."""

    def __init__(self, shape, weights_f32: dict):
        self.lib = ref()
        self.shape = shape
        self._keep = {t: np.ascontiguousarray(a, dtype=np.float32) for t, a in weights_f32.items()}
        ptrs = [self._keep[t].ctypes.data for t in range(12)]
        self.h = self.lib.ref_model_create(shape.dim, shape.hidden_dim, shape.n_layers, shape.n_heads,
                                           shape.n_kv_heads, shape.vocab_size, shape.seq_len, shape.rope_base, *ptrs)
        if not self.h:
            raise MemoryError("ref_model_create failed")

    def close(self):
        if self.h:
            self.lib.ref_model_destroy(self.h)
            self.h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def buf(self, name: str) -> np.ndarray:
        p = self.shape
        kv_dim = p.dim * p.n_kv_heads // p.n_heads
        cache = p.n_layers * p.seq_len * kv_dim
        sizes = {"x": p.dim, "xb": p.dim, "xb2": p.dim, "hb": p.hidden_dim, "he": p.hidden_dim, "q": p.dim,
                 "k": kv_dim, "v": kv_dim, "att": p.n_heads * p.seq_len, "logits": p.vocab_size,
                 "key_cache": cache, "value_cache": cache}
        ptr = self.lib.ref_state_buffer(self.h, STATE_FIELDS.index(name))
        return np.ctypeslib.as_array(ptr, shape=(sizes[name],))

    def forward(self, token, pos, temperature=0.0, topp=1.0, penalty=1.0, history=None) -> int:
        if history is not None and len(history) > 0:
            h = np.ascontiguousarray(history, dtype=np.int32)
            hp, hl = h.ctypes.data, int(h.size)
        else:
            hp, hl = None, 0
        return self.lib.ref_forward(self.h, token, pos, temperature, topp, penalty, hp, hl)
