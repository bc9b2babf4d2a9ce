"""The headline shape at its full size (config 3: Llama-3.2-1B shape, fp16 weights,
and config 4: the same at 8K positions) on a real MI355X.  The oracle needs about a
second per token here, so most checks are properties that do not need it:

  * the three schedules of the library (operator chain, fused graph, persistent
    kernel) are separately written programs over the same weights: their logits must
    agree within the logits bar at every compared position, early, late and at 8K;
  * a run repeated from the same state gives the same bits (the persistent kernel's
    hand-overs carry no arrival-order dependence);
  * the KV cache holds exactly the positions decoded, as binary16 of the run state;
  * a few positions are checked against the oracle directly.
"""
import numpy as np
import pytest

import oracle_binding as ob
from lighterpp_amd import CONFIGS, Model, capi

pytestmark = pytest.mark.gpu
LOGIT_TOL = 2e-3
PATHS = {"ops": capi.PATH_OPS, "fused": capi.PATH_FUSED, "persistent": capi.PATH_PERSISTENT}


def rel_err(got, want):
    want = want.astype(np.float64)
    return float(np.max(np.abs(got.astype(np.float64) - want)) / np.max(np.abs(want)))


@pytest.fixture(scope="module")
def c3():
    shape = CONFIGS["c3_llama32_1b_fp16"]
    m = Model(shape)
    w = m.load_synthetic(1234, keep=True)
    yield shape, m, w
    m.close()


def decode_logits(m, path, tokens, start):
    """Teacher-forced decode of `tokens` from position `start`; logits of every step."""
    m.set_path(path)
    out = []
    for i, t in enumerate(tokens):
        m.forward(int(t), start + i, 0.0)
        out.append(m.buffer(capi.B_LOGITS).copy())
    return out


def test_three_schedules_agree_early_and_late(c3):
    shape, m, _ = c3
    toks = capi.synth_token_ids(24, 3, shape.vocab_size)
    # early: positions 0..23 from an empty cache
    ref = None
    for name, path in PATHS.items():
        m.reset()
        got = decode_logits(m, path, toks, 0)
        if ref is None:
            ref = got
            continue
        worst = max(rel_err(a, b) for a, b in zip(got, ref))
        agree = sum(int(np.argmax(a) == np.argmax(b)) for a, b in zip(got, ref))
        assert worst <= LOGIT_TOL, (name, worst)
        assert agree >= len(toks) - 1, (name, agree)
    # late: fill the cache by generating to position 1500 on the persistent path, then the same
    # eight positions on each schedule over that one cache (a step rewrites only its own slot)
    m.reset()
    m.set_path(capi.PATH_PERSISTENT)
    seq, _, _ = m.generate(int(toks[0]), 0, 1500, temperature=0.0)
    tail = capi.synth_token_ids(8, 9, shape.vocab_size)
    ref = decode_logits(m, capi.PATH_OPS, tail, 1500)
    for name in ("fused", "persistent"):
        got = decode_logits(m, PATHS[name], tail, 1500)
        worst = max(rel_err(a, b) for a, b in zip(got, ref))
        assert worst <= LOGIT_TOL, (name, worst)
    assert len(set(seq.tolist())) > 50, "a 1500-token greedy run over random weights should not collapse"


def test_persistent_run_is_reproducible_bit_for_bit(c3):
    shape, m, _ = c3
    m.set_path(capi.PATH_PERSISTENT)
    u = capi.synth_uniform_f32(160, 5)
    runs = []
    for _ in range(2):
        m.reset()
        toks, hist, _ = m.generate(11, 0, 160, temperature=0.8, penalty=1.1, history_cap=64, uniforms=u)
        runs.append((toks.copy(), list(hist), m.buffer(capi.B_LOGITS).view(np.uint32).copy(),
                     m.buffer(capi.B_KEY_CACHE).copy()))
    assert np.array_equal(runs[0][0], runs[1][0]) and runs[0][1] == runs[1][1]
    assert np.array_equal(runs[0][2], runs[1][2]), "last logits differ between identical runs"
    assert np.array_equal(runs[0][3], runs[1][3]), "key cache differs between identical runs"


def test_cache_holds_exactly_the_decoded_positions(c3):
    shape, m, _ = c3
    hs, nkv, L, S = shape.head_size, shape.n_kv_heads, shape.n_layers, shape.seq_len
    m.reset()
    m.set_path(capi.PATH_PERSISTENT)
    n = 37
    m.generate(7, 0, n, temperature=0.0)
    for b in (capi.B_KEY_CACHE, capi.B_VALUE_CACHE):
        cache = m.buffer(b).reshape(L, nkv, S, hs)
        assert np.all(cache[:, :, n:, :] == 0), "a slot past the decoded positions was written"
        assert np.all(np.any(cache[:, :, :n, :] != 0, axis=-1)), "a decoded position has an empty slot"
    # the run state still holds the last layer's k and v of the last position: the cache has their binary16
    k = m.buffer(capi.B_K).reshape(nkv, hs)
    kc = m.buffer(capi.B_KEY_CACHE).reshape(L, nkv, S, hs)[L - 1, :, n - 1, :]
    assert np.array_equal(kc, capi.f32_to_f16(k.reshape(-1)).reshape(nkv, hs))


def test_persistent_against_oracle_spot_checks(c3):
    shape, m, w = c3
    o = ob.OracleModel(shape, w, fp16=True, kv_round_f16=True)
    m.reset()
    m.set_path(capi.PATH_PERSISTENT)
    tok = 4242
    for pos in range(3):
        nxt = m.forward(tok, pos, 0.0)
        want = o.forward_logits(tok, pos)
        assert rel_err(m.buffer(capi.B_LOGITS), want) <= LOGIT_TOL
        assert nxt == int(np.argmax(want))
        tok = nxt
    o.close()


def test_long_context_schedules_agree_and_match_oracle():
    """Config 4: K/V of positions 0..8191 filled with binary16 N(0,1), decode from 8192."""
    shape = CONFIGS["c4_llama32_1b_longctx_fp16"]
    m = Model(shape)
    w = m.load_synthetic(77, keep=True)
    hs, nkv, L, S = shape.head_size, shape.n_kv_heads, shape.n_layers, shape.seq_len
    start = 8192
    fill = {}
    for b, seed in ((capi.B_KEY_CACHE, 601), (capi.B_VALUE_CACHE, 602)):
        a = capi.synth_normal_f16(L * nkv * S * hs, seed, 1.0).reshape(L, nkv, S, hs)
        a[:, :, start:, :] = 0
        fill[b] = a
    toks = capi.synth_token_ids(4, 21, shape.vocab_size)
    results = {}
    for name, path in PATHS.items():
        for b, a in fill.items():
            m.write_buffer(b, a)
        results[name] = decode_logits(m, path, toks, start)
    for name in ("fused", "persistent"):
        worst = max(rel_err(a, b) for a, b in zip(results[name], results["ops"]))
        assert worst <= LOGIT_TOL, (name, worst)
    # one position against the oracle (its caches are fp32: the same binary16 values, widened)
    o = ob.OracleModel(shape, w, fp16=True, kv_round_f16=True)
    o.buf("key_cache")[:] = capi.f16_to_f32(fill[capi.B_KEY_CACHE].reshape(-1))
    o.buf("value_cache")[:] = capi.f16_to_f32(fill[capi.B_VALUE_CACHE].reshape(-1))
    want = o.forward_logits(int(toks[0]), start)
    assert rel_err(results["persistent"][0], want) <= LOGIT_TOL
    assert int(np.argmax(results["persistent"][0])) == int(np.argmax(want))
    o.close()
    m.close()
