"""The restated oracle must reproduce, bit for bit, what the compiled reference
CPU path produced for the fixtures in tests/golden/ref_cpu_path.npz (written by
tests/golden/make_golden.py from the reference's own ops.cpp + model.cpp).
This is what pins orc_attention / orc_transformer_block / orc_forward /
orc_sample, which no test of the reference covers."""
from pathlib import Path

import numpy as np
import pytest

import oracle_binding as ob
from lighterpp_amd import capi, synth_tensor
from golden.make_golden import CASES, history_push, weights_f32

GOLD = np.load(Path(__file__).parent / "golden" / "ref_cpu_path.npz")
F = np.float32


def bits(a):
    return np.ascontiguousarray(a, dtype=F).view(np.uint32)


def weights_checksum(w):
    c = np.uint64(0)
    for t in range(12):
        c ^= np.bitwise_xor.reduce(w[t].reshape(-1).view(np.uint32).astype(np.uint64) * np.uint64(t + 1))
    return c


@pytest.mark.parametrize("name", list(CASES))
def test_greedy_forward_bit_exact(name):
    shape, seed = CASES[name]
    w = weights_f32(shape, seed)
    if weights_checksum(w) != GOLD[f"{name}/weights_xor"][0]:
        pytest.fail("the synthetic-weight generator no longer reproduces the fixture's inputs")
    prompt = GOLD[f"{name}/prompt"]
    assert np.array_equal(prompt, capi.synth_token_ids(4, seed + 100, shape.vocab_size))
    m = ob.OracleModel(shape, w, fp16=False)
    want_tokens = GOLD[f"{name}/greedy_tokens"]
    want_bits = GOLD[f"{name}/greedy_logit_bits"]
    tok = int(prompt[0])
    for pos in range(len(want_tokens)):
        nxt = m.forward(tok, pos, 0.0, 1.0, 1.0, None, 0.0)
        assert np.array_equal(bits(m.buf("logits")), want_bits[pos]), f"logits differ at pos {pos}"
        assert nxt == want_tokens[pos]
        tok = int(prompt[pos + 1]) if pos + 1 < len(prompt) else nxt
    assert np.array_equal(bits(m.buf("key_cache")), GOLD[f"{name}/key_cache_bits"])
    assert np.array_equal(bits(m.buf("value_cache")), GOLD[f"{name}/value_cache_bits"])
    assert np.array_equal(bits(m.buf("x")), GOLD[f"{name}/x_bits"])
    m.close()


def test_f16_weights_path_equals_widened():
    """The oracle fed binary16 weights directly must equal the oracle (and hence the
    reference) fed the widened copy."""
    name = "gqa8_f16vals"
    shape, seed = CASES[name]
    w16 = {t: synth_tensor(shape, t, seed) for t in range(12)}
    assert w16[2].dtype == np.uint16
    m = ob.OracleModel(shape, w16, fp16=True)
    want_bits = GOLD[f"{name}/greedy_logit_bits"]
    prompt = GOLD[f"{name}/prompt"]
    tok = int(prompt[0])
    for pos in range(len(want_bits)):
        nxt = m.forward(tok, pos, 0.0, 1.0, 1.0, None, 0.0)
        assert np.array_equal(bits(m.buf("logits")), want_bits[pos])
        tok = int(prompt[pos + 1]) if pos + 1 < len(prompt) else nxt
    m.close()


@pytest.mark.parametrize("name", list(CASES))
def test_sampled_run_bit_exact(name):
    shape, seed = CASES[name]
    w = weights_f32(shape, seed)
    m = ob.OracleModel(shape, w, fp16=False)
    draws = GOLD[f"{name}/sampled_draws"]
    want = GOLD[f"{name}/sampled_tokens"]
    prompt = GOLD[f"{name}/prompt"]
    hist = []
    tok = int(prompt[0])
    history_push(hist, 8, tok)
    for pos in range(len(want)):
        nxt = m.forward(tok, pos, 0.8, 1.0, 1.1, hist, float(draws[pos]))
        assert nxt == want[pos], f"token differs at step {pos}"
        tok = nxt
        history_push(hist, 8, tok)
    assert np.array_equal(bits(m.buf("logits")), GOLD[f"{name}/sampled_final_probs_bits"])
    m.close()


def test_sampler_cases_bit_exact():
    base = GOLD["sampler/base_logits"]
    n = int(GOLD["sampler/n"][0])
    assert n >= 20
    for i in range(n):
        win = GOLD[f"sampler/{i}/window"]
        temp, topp, pen, r = (float(v) for v in GOLD[f"sampler/{i}/params"])
        tok, after = ob.orc_sample(base, temp, topp, pen, win, r)
        assert tok == int(GOLD[f"sampler/{i}/token"][0]), f"case {i}"
        assert np.array_equal(bits(after), GOLD[f"sampler/{i}/after_bits"]), f"case {i}"
