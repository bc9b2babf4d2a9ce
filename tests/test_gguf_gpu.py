"""lpp_model_load_gguf on a real MI355X: a model gathered from a GGUF file's named
tensors decodes bit-identically to one whose stacked tensors were uploaded
directly, F32 and F16, tied and untied classifier; what cannot be loaded is
refused with a status."""
import numpy as np
import pytest

import gguf_writer as gw
from lighterpp_amd import Gguf, Model, Shape, capi, synth_tensor

pytestmark = pytest.mark.gpu

CASES = {
    "f32_tied": (Shape(288, 768, 3, 6, 6, 1000, 64, 10000.0, fp16=False, tied=True), False),
    "f32_untied": (Shape(256, 512, 2, 8, 2, 600, 48, 10000.0, fp16=False, tied=False), False),
    "f16_tied_f16_embedding": (Shape(256, 512, 3, 8, 2, 2048, 96, 500000.0, fp16=True, tied=True), True),
    "f16_untied_f32_embedding": (Shape(512, 1024, 2, 4, 2, 777, 48, 500000.0, fp16=True, tied=False), False),
}


@pytest.mark.parametrize("path", [capi.PATH_OPS, capi.PATH_PERSISTENT], ids=["ops", "persistent"])
@pytest.mark.parametrize("name", list(CASES))
def test_model_from_gguf_equals_uploaded_model(name, path, tmp_path):
    shape, f16_embedding = CASES[name]
    w = {t: synth_tensor(shape, t, 17) for t in range(12)}
    file = tmp_path / "model.gguf"
    gw.write_gguf(file, gw.llama_kv(shape), gw.llama_tensors(shape, w, shape.fp16, f16_embedding))
    g = Gguf(file)
    a = Model.from_gguf(g)
    g.close()  # the model holds its own copy in HBM
    assert a.shape.tied == shape.tied and a.shape.fp16 == shape.fp16
    b = Model(shape)
    for t in range(12):
        if t == capi.T_WCLS and shape.tied:
            continue
        b.upload(t, w[t])
    if shape.tied:
        b.tie_classifier()
    for m in (a, b):
        m.set_path(path)
    tok_a = tok_b = 5
    for pos in range(6):
        tok_a = a.forward(tok_a, pos, 0.0)
        la = a.buffer(capi.B_LOGITS)
        tok_b = b.forward(tok_b, pos, 0.0)
        lb = b.buffer(capi.B_LOGITS)
        assert np.array_equal(la.view(np.uint32), lb.view(np.uint32)), f"position {pos}"
        assert tok_a == tok_b
    a.close()
    b.close()


def test_load_refuses_what_it_cannot_hold(tmp_path):
    shape = Shape(64, 160, 2, 8, 2, 96, 48, 10000.0, fp16=True, tied=True)
    w = {t: synth_tensor(shape, t, 3) for t in range(12)}
    kv = gw.llama_kv(shape, noise=False)
    good = gw.llama_tensors(shape, w, True)

    def refuses(tensors, status, match):
        p = tmp_path / "bad.gguf"
        gw.write_gguf(p, kv, tensors)
        g = Gguf(p)
        with pytest.raises(capi.LppError, match=match) as e:
            Model.from_gguf(g)
        assert e.value.status == status
        g.close()

    refuses([t for t in good if t[0] != "blk.1.ffn_up.weight"], capi.LPP_ERR_INVALID_ARG, "missing blk.1.ffn_up")
    refuses([(n, a[:-8], (a.size - 8,)) if n == "blk.0.attn_k.weight" else (n, a, d) for n, a, d in good],
            capi.LPP_ERR_INVALID_ARG, "elements")
    # an F32 matrix in a file whose first matrix is F16 (the reference would upload it with the wrong width)
    refuses([(n, capi.f16_to_f32(a), d) if n == "blk.1.attn_output.weight" else (n, a, d) for n, a, d in good],
            capi.LPP_ERR_UNSUPPORTED, "F32 in a file")
