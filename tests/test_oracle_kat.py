"""Pins the CPU oracle (oracle/lpp_oracle.c) without running any reference code:
the known-answer vectors the reference's own test program holds
(src/runtests.cpp:87-306, restated here as data), closed forms, invariants and
fp64 brute force on small shapes.  Each check is chosen so that a plausible slip
(transposed operand, dropped term, wrong pair convention, wrong GQA mapping)
fails it."""
import ctypes as C

import numpy as np
import pytest

import oracle_binding as ob
from lighterpp_amd import Shape

lib = ob.oracle()
F = np.float32


def f32(*v):
    return np.array(v, dtype=np.float32)


# ---- runtests.cpp known answers -------------------------------------------------

def test_matmul_square_kat():  # runtests.cpp:87-103
    out = np.zeros(2, F)
    lib.orc_naive_matmul(out, f32(1, 2, 3, 4), f32(1, 0, 0, 1), 2, 2)
    assert np.allclose(out, [1.0, 2.0], atol=1e-4)


def test_matmul_rectangular_kat():  # runtests.cpp:105-126; a transposed W would give [2.5, 1, 4][:2]
    out = np.zeros(2, F)
    lib.orc_naive_matmul(out, f32(1, 2, 3), f32(0.5, 0.5, 1.0, 2.0, 0.0, 1.0), 2, 3)
    assert np.allclose(out, [4.5, 5.0], atol=1e-4)


def test_rmsnorm_kat():  # runtests.cpp:128-144
    out = np.zeros(4, F)
    lib.orc_rmsnorm(out, f32(2, 2, 2, 2), f32(1, 1, 1, 1), 4)
    assert np.allclose(out, 1.0, atol=1e-4)


def test_rope_kat():  # runtests.cpp:147-184
    q, k = f32(1, 2, 3, 4), f32(1, 2, 3, 4)
    lib.orc_rope(q, k, 0, 4, 4, 2, 10000.0)
    assert np.array_equal(q, f32(1, 2, 3, 4)) and np.array_equal(k, f32(1, 2, 3, 4))
    q2, k2 = f32(1, 1, 1, 1), f32(1, 1, 1, 1)
    lib.orc_rope(q2, k2, 1, 4, 4, 2, 10000.0)
    assert abs(q2[0] - 1) > 1e-4 and abs(q2[1] - 1) > 1e-4


def test_softmax_kat():  # runtests.cpp:256-283
    x = f32(1, 2, 3)
    lib.orc_softmax(x, 3)
    assert abs(x.sum() - 1) < 1e-4
    assert np.allclose(x, [0.09003, 0.24473, 0.66524], atol=1e-4)


def test_swiglu_kat():  # runtests.cpp:285-306
    hb = np.zeros(2, F)
    lib.orc_swiglu(hb, f32(1, -1), f32(2, 3), 2)
    assert np.allclose(hb, [1.46211, -0.80682], atol=1e-4)


# ---- closed forms and invariants ------------------------------------------------

@pytest.mark.parametrize("n,d", [(7, 13), (64, 288), (33, 2048)])
def test_matmul_fp64_bruteforce(n, d):
    rng = np.random.default_rng(n * 1000 + d)
    x = rng.standard_normal(d).astype(F)
    w = rng.standard_normal((n, d)).astype(F)
    out = np.zeros(n, F)
    lib.orc_naive_matmul(out, x, w.reshape(-1), n, d)
    exact = w.astype(np.float64) @ x.astype(np.float64)
    bound = 2 * d * np.finfo(F).eps * (np.abs(w.astype(np.float64)) @ np.abs(x.astype(np.float64)))
    assert np.all(np.abs(out - exact) <= bound)


def test_matmul_is_sequential_fp32():
    """One fp32 accumulator, k ascending: reproduce the rounding sequence in numpy."""
    rng = np.random.default_rng(3)
    d = 300
    x = rng.standard_normal(d).astype(F)
    w = rng.standard_normal((5, d)).astype(F)
    out = np.zeros(5, F)
    lib.orc_naive_matmul(out, x, w.reshape(-1), 5, d)
    for r in range(5):
        acc = F(0)
        for c in range(d):
            acc = F(acc + F(x[c] * w[r, c]))
        assert out[r] == acc


def test_matmul_f16w_equals_widened():
    rng = np.random.default_rng(4)
    n, d = 19, 136
    wbits = rng.integers(0, 0x7C00, size=n * d, dtype=np.uint16) | (rng.integers(0, 2, n * d, dtype=np.uint16) << 15)
    x = rng.standard_normal(d).astype(F)
    wide = wbits.view(np.float16).astype(F)
    a, b = np.zeros(n, F), np.zeros(n, F)
    lib.orc_matmul_f16w(a, x, wbits, n, d)
    lib.orc_naive_matmul(b, x, wide, n, d)
    assert np.array_equal(a.view(np.uint32), b.view(np.uint32))


def test_f16_widen_exhaustive():
    bits = np.arange(65536, dtype=np.uint16)
    want = bits.view(np.float16).astype(F)
    got = np.array([lib.orc_f16_to_f32(int(b)) for b in bits], dtype=F)
    nan = np.isnan(want)
    assert np.array_equal(np.isnan(got), nan)
    assert np.array_equal(got[~nan].view(np.uint32), want[~nan].view(np.uint32))


def test_f16_narrow_matches_ieee_rn():
    rng = np.random.default_rng(5)
    vals = np.concatenate([
        rng.standard_normal(20000).astype(F) * F(0.02),
        rng.standard_normal(5000).astype(F) * F(300),
        (rng.standard_normal(5000) * 1e-6).astype(F),
        f32(0, -0.0, 65504, 65519.99, 65520, -65520, 1e-8, 5.96e-8, 2.98e-8, 2.9802322e-8, 6.1e-5, 6.0975552e-5),
        np.arange(2048, 2100, dtype=F) + F(0.5),  # exact ties
    ])
    with np.errstate(over="ignore"):
        want = vals.astype(np.float16).view(np.uint16)
    got = np.array([lib.orc_f32_to_f16_rn(float(v)) for v in vals], dtype=np.uint16)
    assert np.array_equal(got, want)


def test_rmsnorm_closed_form():
    rng = np.random.default_rng(6)
    n = 288
    x = rng.standard_normal(n).astype(F)
    g = rng.standard_normal(n).astype(F)
    out = np.zeros(n, F)
    lib.orc_rmsnorm(out, x, g, n)
    exact = x.astype(np.float64) / np.sqrt(np.mean(x.astype(np.float64) ** 2) + 1e-5) * g
    assert np.allclose(out, exact, rtol=1e-5, atol=1e-6)
    inplace = x.copy()
    lib.orc_rmsnorm(inplace, inplace, g, n)  # model.cpp:379 calls it in place
    assert np.array_equal(inplace, out)


@pytest.mark.parametrize("hs,base,pos", [(48, 10000.0, 17), (64, 500000.0, 511), (128, 500000.0, 8447)])
def test_rope_closed_form(hs, base, pos):
    """Adjacent pairs (2i, 2i+1), frequency index 2i mod head_size, k rotated only
    below kv_dim; HF half-split pairing or a per-head restart would fail this."""
    n_heads, n_kv = 4, 2
    dim, kv_dim = hs * n_heads, hs * n_kv
    rng = np.random.default_rng(pos)
    q0 = rng.standard_normal(dim).astype(F)
    k0 = rng.standard_normal(dim).astype(F)  # longer than kv_dim on purpose
    q, k = q0.copy(), k0.copy()
    lib.orc_rope(q, k, pos, dim, kv_dim, hs, base)
    i = np.arange(0, dim, 2)
    # the oracle forms the angle in fp32 (pos * freq); follow that, then rotate in fp64
    # powf is within an ulp of the fp64 power rounded to fp32; an ulp of the
    # frequency moves the angle by up to pos * 2^-23, which the tolerance allows.
    expo = ((i % hs) / F(hs)).astype(F).astype(np.float64)
    freq = (F(1.0) / np.power(np.float64(base), expo).astype(F)).astype(F)
    ang = (F(pos) * freq).astype(F).astype(np.float64)
    c, s = np.cos(ang), np.sin(ang)
    eq = q0[0::2] * c - q0[1::2] * s
    oq = q0[0::2] * s + q0[1::2] * c
    atol = 2e-5 + pos * 2.0 ** -22 * 5
    assert np.allclose(q[0::2], eq, atol=atol) and np.allclose(q[1::2], oq, atol=atol)
    nk = kv_dim // 2
    assert np.allclose(k[0:kv_dim:2], k0[0:kv_dim:2] * c[:nk] - k0[1:kv_dim:2] * s[:nk], atol=atol)
    assert np.array_equal(k[kv_dim:], k0[kv_dim:])  # untouched beyond kv_dim
    # rotation preserves each pair's norm
    assert np.allclose(q[0::2] ** 2 + q[1::2] ** 2, q0[0::2] ** 2 + q0[1::2] ** 2, rtol=1e-5)


def test_rope_composes():
    """R(a) then R(b) on the angles of positions a and b equals R(a+b) when the
    angles add exactly: use base 1 so every frequency is 1 and angle = pos."""
    hs, dim = 8, 16
    rng = np.random.default_rng(8)
    q0 = rng.standard_normal(dim).astype(F)
    k0 = np.zeros(dim, F)
    a = q0.copy()
    lib.orc_rope(a, k0.copy(), 3, dim, 0, hs, 1.0)
    lib.orc_rope(a, k0.copy(), 4, dim, 0, hs, 1.0)
    b = q0.copy()
    lib.orc_rope(b, k0.copy(), 7, dim, 0, hs, 1.0)
    assert np.allclose(a, b, atol=1e-5)


def test_softmax_properties():
    rng = np.random.default_rng(9)
    x = (rng.standard_normal(1000) * 5).astype(F)
    a = x.copy()
    lib.orc_softmax(a, a.size)
    exact = np.exp(x.astype(np.float64) - x.max())
    exact /= exact.sum()
    assert np.allclose(a, exact, rtol=2e-5, atol=1e-9)
    b = (x + F(8)).astype(F)  # shift by a power of two: exactly representable differences
    lib.orc_softmax(b, b.size)
    assert np.allclose(a, b, rtol=1e-5)
    one = f32(3.5)
    lib.orc_softmax(one, 1)
    assert one[0] == 1.0


def test_swiglu_closed_form_and_alias():
    rng = np.random.default_rng(10)
    g = (rng.standard_normal(500) * 3).astype(F)
    u = rng.standard_normal(500).astype(F)
    out = np.zeros(500, F)
    lib.orc_swiglu(out, g, u, 500)
    exact = g.astype(np.float64) / (1 + np.exp(-g.astype(np.float64))) * u
    assert np.allclose(out, exact, rtol=1e-5, atol=1e-7)
    alias = g.copy()
    lib.orc_swiglu(alias, alias, u, 500)  # model.cpp:237 passes hb as both
    assert np.array_equal(alias, out)


# ---- attention / block / forward against fp64 numpy ------------------------------

def rand_weights(shape: Shape, seed: int) -> dict:
    rng = np.random.default_rng(seed)
    w = {}
    for t in range(12):
        dims = shape.tensor_shape(t)
        scale = 1.0 if t in (1, 6, 10) else 0.2
        a = rng.standard_normal(dims) * scale
        if t in (1, 6, 10):
            a = 1.0 + 0.1 * a
        w[t] = a.astype(F)
    return w


def numpy_forward(shape: Shape, w: dict, tokens, dtype=np.float64):
    """Independent fp64 statement of the Llama decode step in the reference's
    conventions (interleaved RoPE, GQA head h -> kv head h // group,
    cache [layer][kv_head][pos][hs])."""
    d, hs, nh, nkv = shape.dim, shape.head_size, shape.n_heads, shape.n_kv_heads
    group = nh // nkv
    W = {t: a.astype(dtype) for t, a in w.items()}
    kc = np.zeros((shape.n_layers, nkv, shape.seq_len, hs), dtype)
    vc = np.zeros_like(kc)
    outs = []

    def norm(x, g):
        return x / np.sqrt(np.mean(x * x) + 1e-5) * g

    def rope(vec, pos, nheads):
        v = vec.reshape(nheads, hs // 2, 2).copy()
        idx = np.arange(0, hs, 2)
        freq = (np.float32(1.0) / np.power(np.float32(shape.rope_base), (idx / np.float32(hs)).astype(np.float32))
                ).astype(np.float32)
        ang = (np.float32(pos) * freq).astype(np.float32).astype(dtype)
        c, s = np.cos(ang), np.sin(ang)
        a, b = v[..., 0].copy(), v[..., 1].copy()
        v[..., 0] = a * c - b * s
        v[..., 1] = a * s + b * c
        return v.reshape(-1)

    for pos, tok in enumerate(tokens):
        x = W[0][tok].copy()
        for l in range(shape.n_layers):
            xb = norm(x, W[1][l])
            q = rope(W[2][l] @ xb, pos, nh)
            k = rope(W[3][l] @ xb, pos, nkv)
            v = W[4][l] @ xb
            kc[l, :, pos] = k.reshape(nkv, hs)
            vc[l, :, pos] = v.reshape(nkv, hs)
            att_out = np.zeros(d, dtype)
            for h in range(nh):
                kvh = h // group
                sc = kc[l, kvh, :pos + 1] @ q[h * hs:(h + 1) * hs] / np.sqrt(np.float32(hs))
                p = np.exp(sc - sc.max())
                p /= p.sum()
                att_out[h * hs:(h + 1) * hs] = p @ vc[l, kvh, :pos + 1]
            x = x + W[5][l] @ att_out
            xb = norm(x, W[6][l])
            g, u = W[7][l] @ xb, W[9][l] @ xb
            x = x + W[8][l] @ (g / (1 + np.exp(-g)) * u)
        outs.append(W[11] @ norm(x, W[10]))
    return np.array(outs), kc, vc


@pytest.mark.parametrize("nh,nkv", [(4, 4), (8, 2), (8, 1)])
def test_forward_matches_fp64_numpy(nh, nkv):
    hs = 8
    shape = Shape(nh * hs, 96, 2, nh, nkv, 50, 12, 10000.0, fp16=False, tied=False)
    w = rand_weights(shape, 100 + nh + nkv)
    tokens = [3, 17, 42, 8, 8, 0, 49]
    m = ob.OracleModel(shape, w, fp16=False)
    got = np.array([m.forward_logits(t, p) for p, t in enumerate(tokens)])
    want, kc, vc = numpy_forward(shape, w, tokens)
    assert np.allclose(got, want, rtol=2e-4, atol=2e-4)
    # KV scatter layout: cache[layer][kv_head][pos][i]
    got_k = m.buf("key_cache").reshape(shape.n_layers, nkv, shape.seq_len, hs)
    assert np.allclose(got_k[:, :, :len(tokens)], kc[:, :, :len(tokens)], rtol=2e-4, atol=2e-4)
    assert np.all(got_k[:, :, len(tokens):] == 0)
    m.close()


def test_kv_scatter_index_exhaustive():
    """model.cpp:173: dst = layer*(kv_dim*seq_len) + head*(seq_len*hs) + pos*hs + i.
    Identity-like weights make k equal to a known pattern, so every written slot can
    be predicted exactly."""
    hs, nh, nkv, L, seq = 4, 4, 2, 3, 5
    dim, kv_dim = nh * hs, nkv * hs
    shape = Shape(dim, 8, L, nh, nkv, 10, seq, 10000.0, fp16=False, tied=False)
    w = {t: np.zeros(shape.tensor_shape(t), F) for t in range(12)}
    for t in (1, 6, 10):
        w[t][:] = 1
    sel = np.zeros((kv_dim, dim), F)
    sel[np.arange(kv_dim), np.arange(kv_dim)] = 1
    for l in range(L):
        w[4][l] = sel * (l + 1)          # v = (l+1) * xb[:kv_dim], no RoPE on v
    m = ob.OracleModel(shape, w, fp16=False)
    xb = np.arange(1, dim + 1, dtype=F)
    for pos in range(seq):
        for l in range(L):
            m.buf("xb")[:] = xb * (pos + 1)
            m.attention(l, pos)
    vc = m.buf("value_cache")
    for l in range(L):
        for h in range(nkv):
            for pos in range(seq):
                for i in range(hs):
                    idx = l * (kv_dim * seq) + h * (seq * hs) + pos * hs + i
                    assert vc[idx] == (l + 1) * (pos + 1) * xb[h * hs + i]
    m.close()


def test_kv_round_f16_switch():
    shape = Shape(32, 64, 1, 4, 2, 20, 6, 10000.0, fp16=False, tied=False)
    w = rand_weights(shape, 77)
    a = ob.OracleModel(shape, w, fp16=False, kv_round_f16=False)
    b = ob.OracleModel(shape, w, fp16=False, kv_round_f16=True)
    a.forward_logits(5, 0)
    b.forward_logits(5, 0)
    ka, kb = a.buf("key_cache"), b.buf("key_cache")
    assert np.array_equal(kb, ka.astype(np.float16).astype(F))
    assert not np.array_equal(ka, kb)
    a.close()
    b.close()


# ---- sampler -----------------------------------------------------------------------

def py_sample(logits, temperature, penalty, history, r):
    """model.cpp:256-303 in exact fp32 steps (plain-CDF branch)."""
    lg = logits.astype(F).copy()
    n = lg.size
    if penalty > 1.0 and history is not None and len(history) > 0:
        for t in history:
            if 0 <= t < n:
                lg[t] = F(lg[t] / F(penalty)) if lg[t] > 0 else F(lg[t] * F(penalty))
    if temperature == 0.0:
        return int(np.argmax(lg)), lg  # numpy argmax returns the first maximum
    lg = (lg / F(temperature)).astype(F)
    mx = lg.max()
    e = np.exp((lg - mx).astype(F)).astype(F)  # numpy expf may differ by an ulp from libm; checked loosely
    return None, e


def test_sampler_penalty_per_occurrence_and_sign():
    lg = f32(2.0, -2.0, 0.0, 1.0, 5.0)
    tok, after = ob.orc_sample(lg, 0.0, 1.0, 2.0, [0, 0, 1, 1, 1, 2, 7, -1], 0.0)
    # token 0 twice: 2/2/2; token 1 three times: -2*2*2*2; token 2 (== 0, not > 0): 0*2
    assert np.array_equal(after, f32(0.5, -16.0, 0.0, 1.0, 5.0))
    assert tok == 4
    # penalty <= 1 is a no-op (model.cpp:259)
    _, untouched = ob.orc_sample(lg, 0.0, 1.0, 1.0, [0, 0, 1], 0.0)
    assert np.array_equal(untouched, lg)


def test_sampler_argmax_first_max_wins():
    lg = f32(1, 7, 3, 7, 7, -2)
    assert ob.orc_sample(lg, 0.0, 1.0, 1.0, None, 0.0)[0] == 1
    # penalty can demote the first maximum
    assert ob.orc_sample(lg, 0.0, 1.0, 1.5, [1], 0.0)[0] == 3


def test_sampler_cdf_edges():
    lg = np.log(f32(0.1, 0.2, 0.3, 0.4))
    probs = ob.orc_sample(lg, 1.0, 1.0, 1.0, None, 0.5)[1]
    cdf = np.cumsum(probs.astype(np.float64))
    for r, want in [(0.0, 0), (0.0999, 0), (0.1001, 1), (0.2999, 1), (0.3001, 2), (0.5999, 2), (0.6001, 3),
                    (0.99999, 3)]:
        assert ob.orc_sample(lg, 1.0, 1.0, 1.0, None, r)[0] == want
    # r >= total mass falls through to vocab-1 (model.cpp:302)
    assert ob.orc_sample(lg, 1.0, 1.0, 1.0, None, 1.0)[0] == 3
    assert abs(cdf[-1] - 1) < 1e-6
    # r is compared with strict <: r exactly on an edge goes to the next bucket
    two = f32(0.0, 0.0)
    assert ob.orc_sample(two, 1.0, 1.0, 1.0, None, 0.5)[0] == 1
    assert ob.orc_sample(two, 1.0, 1.0, 1.0, None, np.nextafter(F(0.5), F(0)))[0] == 0


def test_sampler_temperature_divides():
    lg = f32(1.0, 2.0, 4.0)
    a = ob.orc_sample(lg, 0.5, 1.0, 1.0, None, 0.0)[1]
    exact = np.exp(np.array([2.0, 4.0, 8.0]) - 8.0)
    exact /= exact.sum()
    assert np.allclose(a, exact, rtol=1e-5)


def test_sampler_bruteforce_distribution():
    """Every r on a fine grid lands in the bucket the fp64 CDF predicts, except
    within 1e-5 of an edge."""
    rng = np.random.default_rng(11)
    lg = (rng.standard_normal(50) * 2).astype(F)
    hist = [3, 3, 9, 20, 49]
    pen, temp = 1.2, 0.8
    ref = lg.astype(np.float64).copy()
    for t in hist:
        ref[t] = ref[t] / pen if ref[t] > 0 else ref[t] * pen
    p = np.exp(ref / temp - (ref / temp).max())
    p /= p.sum()
    cdf = np.cumsum(p)
    for r in np.linspace(0, 0.9999, 400):
        tok = ob.orc_sample(lg, temp, 1.0, pen, hist, float(F(r)))[0]
        want = int(np.searchsorted(cdf, float(F(r)), side="right"))
        if np.min(np.abs(cdf - float(F(r)))) > 1e-5:
            assert tok == min(want, 49)


def test_sample_cdf_reports_bucket():
    lg = np.log(f32(0.25, 0.25, 0.5))
    tok, lo, hi = ob.orc_sample_cdf(lg, 1.0, 1.0, None, 0.3)
    assert tok == 1 and abs(lo - 0.25) < 1e-6 and abs(hi - 0.5) < 1e-6


def test_history_push_window():  # main.cpp:203-208
    h = np.zeros(4, np.int32)
    n = C.c_int(0)
    for t in range(1, 7):
        lib.orc_history_push(h, C.byref(n), 4, t)
    assert n.value == 4 and h.tolist() == [3, 4, 5, 6]
