"""The reference's own forward() (src/model.cpp:342-371, USE_CUDA branch: its 404 operator launches per token)
running on the MI355X through include/lpp_kernels_compat.h and liblpp_hip.so, against the CPU oracle.
oracle/_ref/libref_on_lpp.so is built on the CPU side from the reference's sources (tests/dropin/Makefile);
skipped where it is absent."""
import ctypes as C
from pathlib import Path

import numpy as np
import pytest

import oracle_binding as ob
from lighterpp_amd import Shape, capi
from lighterpp_amd.model import synth_tensor

pytestmark = pytest.mark.gpu
ROOT = Path(__file__).resolve().parents[1]
LIB = ROOT / "oracle" / "_ref" / "libref_on_lpp.so"

SHAPES = {
    "gqa4_fp16": Shape(256, 512, 3, 8, 2, 2048, 160, 500000.0, fp16=True, tied=True),
    "mha_fp32": Shape(288, 768, 2, 6, 6, 1000, 64, 10000.0, fp16=False, tied=True),
}


@pytest.mark.skipif(not LIB.exists(), reason="oracle/_ref/libref_on_lpp.so not built (needs the reference's sources)")
@pytest.mark.parametrize("name", list(SHAPES))
def test_reference_forward_runs_on_the_library(name):
    shape = SHAPES[name]
    capi.check(capi.load().lpp_init(0))
    ref = C.CDLL(str(LIB))
    ref.rol_create.restype = C.c_void_p
    ref.rol_create.argtypes = [C.c_int] * 7 + [C.c_float, C.c_int]
    ref.rol_upload.argtypes = [C.c_void_p, C.c_int, C.c_void_p, C.c_size_t]
    ref.rol_forward.argtypes = [C.c_void_p, C.c_int, C.c_int, C.c_void_p]
    ref.rol_destroy.argtypes = [C.c_void_p]
    h = ref.rol_create(shape.dim, shape.hidden_dim, shape.n_layers, shape.n_heads, shape.n_kv_heads, shape.vocab_size,
                       shape.seq_len, shape.rope_base, capi.WEIGHT_FP16 if shape.fp16 else capi.WEIGHT_FP32)
    weights = {}
    for t in range(12):
        if t == capi.T_WCLS:  # tied: the classifier is the embedding, narrowed for binary16 models (loader.cpp:619-632)
            emb = weights[capi.T_TOKEN_EMBEDDING]
            a = capi.f32_to_f16(emb).reshape(emb.shape) if shape.fp16 else emb
        else:
            a = synth_tensor(shape, t, 4)
        weights[t] = a
        a = np.ascontiguousarray(a)
        assert ref.rol_upload(h, t, C.c_void_p(a.ctypes.data), a.nbytes) == 0
    o = ob.OracleModel(shape, weights, fp16=shape.fp16, kv_round_f16=True)
    logits = np.empty(shape.vocab_size, np.float32)
    tok = 5
    for pos in range(8):
        nxt = ref.rol_forward(h, tok, pos, C.c_void_p(logits.ctypes.data))
        want = o.forward_logits(tok, pos)
        err = float(np.max(np.abs(logits.astype(np.float64) - want)) / np.max(np.abs(want)))
        assert err <= 2e-3, (pos, err)
        assert nxt == int(np.argmax(want)), pos
        tok = nxt
    ref.rol_destroy(h)
    o.close()
