"""Live comparison of the restated oracle with the compiled reference
(oracle/_ref/liblpp_ref.so), wherever that library exists (it is built in the
container that holds the reference sources and travels as a binary).  Random
shapes and inputs beyond the committed fixtures; everything must be bit-equal."""
import numpy as np
import pytest

import oracle_binding as ob
from lighterpp_amd import Shape
from test_oracle_kat import rand_weights

pytestmark = pytest.mark.skipif(not ob.have_ref(), reason="oracle/_ref/liblpp_ref.so not built")
F = np.float32


def bits(a):
    return np.ascontiguousarray(a, dtype=F).view(np.uint32)


@pytest.mark.parametrize("seed", range(4))
def test_ops_bit_equal(seed):
    rng = np.random.default_rng(seed)
    lib, ref = ob.oracle(), ob.ref()
    n, d = int(rng.integers(1, 70)), int(rng.integers(1, 400))
    x = rng.standard_normal(d).astype(F)
    w = rng.standard_normal(n * d).astype(F)
    a, b = np.zeros(n, F), np.zeros(n, F)
    lib.orc_naive_matmul(a, x, w, n, d)
    ref.ref_naive_matmul(b, x.copy(), w.copy(), n, d)
    assert np.array_equal(bits(a), bits(b))

    g = rng.standard_normal(d).astype(F)
    a, b = np.zeros(d, F), np.zeros(d, F)
    lib.orc_rmsnorm(a, x, g, d)
    ref.ref_rmsnorm(b, x.copy(), g.copy(), d)
    assert np.array_equal(bits(a), bits(b))

    hs = int(rng.choice([2, 8, 48, 64, 128]))
    nh, nkv = 4, int(rng.choice([1, 2, 4]))
    dim, kv_dim = hs * nh, hs * nkv
    pos = int(rng.integers(0, 9000))
    base = float(rng.choice([10000.0, 500000.0]))
    q = rng.standard_normal(dim).astype(F)
    k = rng.standard_normal(dim).astype(F)
    qa, ka, qb, kb = q.copy(), k.copy(), q.copy(), k.copy()
    lib.orc_rope(qa, ka, pos, dim, kv_dim, hs, base)
    ref.ref_rope(qb, kb, pos, dim, kv_dim, hs, base)
    assert np.array_equal(bits(qa), bits(qb)) and np.array_equal(bits(ka), bits(kb))

    s = (rng.standard_normal(d) * 4).astype(F)
    sa, sb = s.copy(), s.copy()
    lib.orc_softmax(sa, d)
    ref.ref_softmax(sb, d)
    assert np.array_equal(bits(sa), bits(sb))

    h3 = rng.standard_normal(d).astype(F)
    a, b = np.zeros(d, F), np.zeros(d, F)
    lib.orc_swiglu(a, s, h3, d)
    ref.ref_swiglu(b, s.copy(), h3.copy(), d)
    assert np.array_equal(bits(a), bits(b))


@pytest.mark.parametrize("nh,nkv,hs", [(6, 6, 48), (8, 2, 16), (8, 1, 8)])
def test_forward_bit_equal(nh, nkv, hs):
    shape = Shape(nh * hs, 3 * nh * hs // 2, 2, nh, nkv, 300, 16, 500000.0, fp16=False, tied=False)
    w = rand_weights(shape, nh * 100 + nkv)
    o = ob.OracleModel(shape, w, fp16=False)
    r = ob.RefModel(shape, w)
    lib = ob.ref()
    lib.ref_srand(99)
    draws = [lib.ref_next_uniform() for _ in range(16)]
    lib.ref_srand(99)
    hist = [7]
    tok = 7
    for pos in range(16):
        a = o.forward(tok, pos, 0.9, 1.0, 1.15, hist, draws[pos])
        b = r.forward(tok, pos, 0.9, 1.0, 1.15, hist)
        assert a == b, f"step {pos}"
        assert np.array_equal(bits(o.buf("logits")), bits(r.buf("logits")))
        for name in ("x", "q", "k", "v", "hb", "key_cache", "value_cache", "att"):
            assert np.array_equal(bits(o.buf(name)), bits(r.buf(name))), name
        tok = a
        hist = (hist + [tok])[-4:]
    o.close()
    r.close()


def test_nucleus_branch_bit_equal():
    rng = np.random.default_rng(5)
    lib = ob.ref()
    for case in range(20):
        lg = (rng.standard_normal(333) * 2).astype(F)
        topp = float(rng.uniform(0.05, 0.95))
        lib.ref_srand(case)
        r = lib.ref_next_uniform()
        lib.ref_srand(case)
        mine = lg.copy()
        want = lib.ref_sample(mine, mine.size, 1.1, topp, 1.0, None, 0)
        got, after = ob.orc_sample(lg, 1.1, topp, 1.0, None, r)
        assert got == want and np.array_equal(bits(after), bits(mine))
