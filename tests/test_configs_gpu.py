"""Every benchmark configuration at its full shape against the CPU oracle on a real
MI355X, on the schedule the benchmark runs (the persistent kernel) and on the fused
graph: config 1 for all of its 256 positions, config 2 (TinyLlama shape: 22 layers,
4 KV heads under 32 query heads, untied classifier) through its 16 prompt ids and
16 decode steps, config 3's own workload (temperature 0.8, penalty 1.1, 64-entry
window, seeded draws) plus 64 teacher-forced greedy steps, and config 5 (Llama-3-8B
shape: head size 128, 14336 hidden units cut into column slices).  Config 4 (8K
positions) is in test_full_size_gpu.py.

Bars: max |gpu - cpu| / max |cpu| <= 2e-3 per step; greedy ids agree on >= 99 % of
steps; a sampled id may differ only where the draw sits within the logits tolerance
of an edge of the CPU's cumulative distribution; cache slots bit-exact binary16 of
the run state.  The oracle is teacher-forced (both sides get the oracle's token, or
the GPU's sampled one), so one allowed flip cannot cascade.
"""
import numpy as np
import pytest

import oracle_binding as ob
from lighterpp_amd import CONFIGS, Model, capi

pytestmark = pytest.mark.gpu
LOGIT_TOL = 2e-3
FAST = {"fused": capi.PATH_FUSED, "persistent": capi.PATH_PERSISTENT}
ALL = {"ops": capi.PATH_OPS, **FAST}


def rel_err(got, want):
    want = want.astype(np.float64)
    return float(np.max(np.abs(got.astype(np.float64) - want)) / np.max(np.abs(want)))


def teacher_forced(m, o, paths, tokens_in, n_steps, start=0):
    """Feeds prompt ids, then the oracle's own greedy ids, to the oracle once and to every
    path; returns per path (worst logit error, greedy agreements) and the ids fed."""
    want_logits, fed = [], []
    tok = int(tokens_in[0])
    for i in range(n_steps):
        fed.append(tok)
        want = o.forward_logits(tok, start + i)
        want_logits.append(want)
        tok = int(tokens_in[i + 1]) if i + 1 < len(tokens_in) else int(np.argmax(want))
    out = {}
    for name, path in paths.items():
        m.reset()
        m.set_path(path)
        worst, agree = 0.0, 0
        for i, t in enumerate(fed):
            nxt = m.forward(t, start + i, 0.0)
            worst = max(worst, rel_err(m.buffer(capi.B_LOGITS), want_logits[i]))
            agree += int(nxt == int(np.argmax(want_logits[i])))
        out[name] = (worst, agree)
    return out, fed


def assert_last_slot_is_run_state(m, shape, pos):
    hs, nkv, L, S = shape.head_size, shape.n_kv_heads, shape.n_layers, shape.seq_len
    for buf, cache in ((capi.B_K, capi.B_KEY_CACHE), (capi.B_V, capi.B_VALUE_CACHE)):
        vec = m.buffer(buf)
        got = m.buffer(cache).reshape(L, nkv, S, hs)
        assert np.array_equal(got[L - 1, :, pos, :], capi.f32_to_f16(vec).reshape(nkv, hs))
        assert not got[:, :, pos + 1:, :].any(), "a slot past the decoded positions was written"
        assert np.all(np.any(got[:, :, :pos + 1, :] != 0, axis=-1)), "a decoded position has an empty slot"


def test_c1_all_256_positions():
    """Config 1 (llama2.c 15M, fp32): 8 prompt ids, then greedy to the end of the context."""
    shape = CONFIGS["c1_llama2c_15m_fp32"]
    m = Model(shape)
    w = m.load_synthetic(1234, keep=True)
    o = ob.OracleModel(shape, w, fp16=False, kv_round_f16=True)
    prompt = capi.synth_token_ids(8, 77, shape.vocab_size)
    res, fed = teacher_forced(m, o, FAST, prompt, shape.seq_len)
    for name, (worst, agree) in res.items():
        print(f"c1 {name}: max rel logit err {worst:.2e}, greedy {agree}/{shape.seq_len}", flush=True)
        assert worst <= LOGIT_TOL, (name, worst)
        assert agree >= int(np.ceil(0.99 * shape.seq_len)), (name, agree)
    assert_last_slot_is_run_state(m, shape, shape.seq_len - 1)
    # free-running greedy generation on the persistent path reproduces the oracle's ids
    m.reset()
    m.set_path(capi.PATH_PERSISTENT)
    for i in range(7):
        m.forward(int(prompt[i]), i, 0.0)
    toks, _, _ = m.generate(int(prompt[7]), 7, shape.seq_len - 7, temperature=0.0)
    same = np.mean(np.array(fed[8:]) == toks[:len(fed) - 8])
    assert same >= 0.99, same
    m.close()
    o.close()


@pytest.mark.timeout(600)
def test_c2_tinyllama_shape_prompt_and_decode():
    """Config 2: 22 layers, 8 query heads per KV head, untied classifier, rope base 1e4."""
    shape = CONFIGS["c2_tinyllama_1b_fp16"]
    m = Model(shape)
    w = m.load_synthetic(1234, keep=True)
    o = ob.OracleModel(shape, w, fp16=True, kv_round_f16=True)
    prompt = capi.synth_token_ids(16, 77, shape.vocab_size)
    steps = 32
    res, _ = teacher_forced(m, o, ALL, prompt, steps)
    for name, (worst, agree) in res.items():
        print(f"c2 {name}: max rel logit err {worst:.2e}, greedy {agree}/{steps}", flush=True)
        assert worst <= LOGIT_TOL, (name, worst)
        assert agree >= int(np.ceil(0.99 * steps)), (name, agree)
    assert_last_slot_is_run_state(m, shape, steps - 1)
    m.close()
    o.close()


@pytest.mark.timeout(600)
def test_c3_sampled_workload_and_greedy_agreement():
    """Config 3 as the benchmark runs it, on the persistent kernel."""
    shape = CONFIGS["c3_llama32_1b_fp16"]
    m = Model(shape)
    w = m.load_synthetic(1234, keep=True)
    o = ob.OracleModel(shape, w, fp16=True, kv_round_f16=True)
    m.set_path(capi.PATH_PERSISTENT)
    steps, first = 40, 4242
    draws = capi.synth_uniform_f32(steps, 99)
    toks, hist_after, _ = m.generate(first, 0, steps, temperature=0.8, penalty=1.1, history=[first], history_cap=64,
                                     uniforms=draws)
    # At 128 K near-uniform entries a bucket of the cumulative distribution is ~1e-5 wide, as wide as the
    # drift of the CPU's own running fp32 sum: ids differ from the CPU sampler's often, and what is pinned is
    # WHERE the GPU's id sits -- (a) the draw within the logits tolerance of an edge of the CPU's bucket, and
    # (b) inside the id's own bucket of the float64 distribution over the CPU's logits, to 2e-4 (a sampler
    # that walked the vocabulary in another order, or dropped a chunk's mass, is off by orders more).
    hist, tok, flips, worst64 = [first], first, 0, 0.0
    for i in range(steps):
        o.forward_logits(tok, i)
        r = float(draws[i])
        want, lo, hi = ob.orc_sample_cdf(o.buf("logits"), 0.8, 1.1, hist, r)
        if toks[i] != want:
            flips += 1
            gap = min(abs(r - lo), abs(r - hi))
            assert gap < LOGIT_TOL, f"step {i}: token {toks[i]} vs {want}, CDF gap {gap}"
        _, penalised = ob.orc_sample(o.buf("logits"), 0.0, 1.0, 1.1, hist, 0.0)  # the penalty step alone
        z = penalised.astype(np.float64) / np.float64(np.float32(0.8))
        p = np.exp(z - z.max())
        p /= p.sum()
        lo64 = float(p[:toks[i]].sum())
        off = max(lo64 - r, r - (lo64 + float(p[toks[i]])), 0.0)
        worst64 = max(worst64, off)
        assert off <= 2e-4, f"step {i}: draw {r} is {off} outside the float64 bucket of id {toks[i]}"
        tok = int(toks[i])
        hist = (hist + [tok])[-64:]
    print(f"c3 sampled: {steps} steps, {flips} ids differ from the CPU sampler's (each within the CDF gap); "
          f"draw at most {worst64:.1e} outside the id's float64 bucket", flush=True)
    assert hist_after == hist
    # greedy, teacher-forced: 64 steps so that "99 % of steps" is measured on more than a handful
    o2 = ob.OracleModel(shape, w, fp16=True, kv_round_f16=True)
    res, _ = teacher_forced(m, o2, {"persistent": capi.PATH_PERSISTENT}, [first], 64)
    worst, agree = res["persistent"]
    print(f"c3 greedy persistent: max rel logit err {worst:.2e}, greedy {agree}/64", flush=True)
    assert worst <= LOGIT_TOL and agree >= 64
    m.close()
    o.close()
    o2.close()


@pytest.mark.timeout(900)
def test_c5_llama3_8b_shape():
    """Config 5: head size 128, hidden 14336 (seven column slices per down-projection row)."""
    shape = CONFIGS["c5_llama3_8b_fp16"]
    print("c5: generating 7.5 G synthetic weights", flush=True)
    m = Model(shape)
    w = m.load_synthetic(1234, keep=True)
    o = ob.OracleModel(shape, w, fp16=True, kv_round_f16=True)
    prompt = capi.synth_token_ids(2, 77, shape.vocab_size)
    steps = 4
    res, fed = teacher_forced(m, o, ALL, prompt, steps)
    for name, (worst, agree) in res.items():
        print(f"c5 {name}: max rel logit err {worst:.2e}, greedy {agree}/{steps}", flush=True)
        assert worst <= LOGIT_TOL, (name, worst)
        assert agree >= int(np.ceil(0.99 * steps)), (name, agree)
    assert_last_slot_is_run_state(m, shape, steps - 1)
    # the persistent kernel repeats bit for bit
    m.set_path(capi.PATH_PERSISTENT)
    runs = []
    for _ in range(2):
        m.reset()
        toks, _, _ = m.generate(int(fed[0]), 0, 24, temperature=0.0)
        runs.append((toks.copy(), m.buffer(capi.B_LOGITS).view(np.uint32).copy(), m.buffer(capi.B_KEY_CACHE).copy()))
    assert np.array_equal(runs[0][0], runs[1][0])
    assert np.array_equal(runs[0][1], runs[1][1]) and np.array_equal(runs[0][2], runs[1][2])
    m.close()
    o.close()
