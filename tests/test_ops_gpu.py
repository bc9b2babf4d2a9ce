"""Parity of the twelve operator entry points (include/lpp.h section A, the
surface of the reference's src/kernels.cuh:24-36) against the CPU oracle, called
through the C ABI on a real MI355X.

Inputs restate the patterned vectors of the reference's CUDA-vs-CPU tests
(src/runtests.cpp:313-875) and add seeded random shapes from the five benchmark
configurations plus ragged / misaligned / tiny edge cases.

Bars: integer, byte and index work (f32->f16 cast, KV scatter, argmax, residual
add, RoPE with host-built tables) bit-exact; floating point within the
tolerance written beside each assert, all far inside the 2e-3 the logits are
allowed."""
import ctypes as C

import numpy as np
import pytest

import oracle_binding as ob
from lighterpp_amd import capi
from lighterpp_amd.capi import DeviceBuffer as DB

pytestmark = pytest.mark.gpu
F = np.float32
orc = ob.oracle()


@pytest.fixture(scope="module")
def lib():
    lib = capi.load()
    assert capi.device_count() >= 1, "no HIP device visible"
    capi.check(lib.lpp_init(0))
    return lib


def bits(a):
    return np.ascontiguousarray(a, dtype=F).view(np.uint32)


def gemv_gpu(lib, x, w, n, d, precision):
    dx, dw, dout = DB.from_numpy(x), DB.from_numpy(w), DB(max(n, 1) * 4)
    capi.check(lib.lpp_gemv(dout.ptr, dx.ptr, dw.ptr, None, n, d, precision))
    return dout.to_numpy(F, n)


# ---- gemv -------------------------------------------------------------------------

def test_gemv_fp32_runtests_pattern(lib):  # runtests.cpp:313-383
    n, d = 256, 512
    x = (0.1 * (np.arange(d) % 10)).astype(F)
    w = (0.01 * (np.arange(n * d) % 100)).astype(F)
    want = np.zeros(n, F)
    orc.orc_naive_matmul(want, x, w, n, d)
    got = gemv_gpu(lib, x, w, n, d, capi.WEIGHT_FP32)
    assert np.max(np.abs(got - want)) < 1e-3  # the reference's own bar (runtests.cpp:83-85)
    assert np.max(np.abs(got - want) / np.abs(want).max()) < 2e-6


def test_gemv_fp16_runtests_pattern(lib):  # runtests.cpp:385-469: weights cast on the device
    n, d = 256, 512
    x = (0.1 * (np.arange(d) % 10)).astype(F)
    w = (0.01 * (np.arange(n * d) % 100)).astype(F)
    dw32, dw16 = DB.from_numpy(w), DB(n * d * 2)
    capi.check(lib.lpp_convert_f32_to_f16(dw16.ptr, dw32.ptr, n * d))
    w16 = dw16.to_numpy(np.uint16)
    assert np.array_equal(w16, w.astype(np.float16).view(np.uint16))  # RN cast, bit-exact
    want = np.zeros(n, F)
    orc.orc_matmul_f16w(want, x, w16, n, d)
    dx, dout = DB.from_numpy(x), DB(n * 4)
    capi.check(lib.lpp_gemv(dout.ptr, dx.ptr, dw16.ptr, None, n, d, capi.WEIGHT_FP16))
    got = dout.to_numpy(F)
    assert np.all(np.abs(got - want) <= np.abs(want) * 0.01 + 1e-4)  # reference bar (runtests.cpp:451)
    assert np.max(np.abs(got - want) / np.abs(want).max()) < 2e-6    # ours: fp32 accumulate


GEMV_SHAPES = [
    (288, 288), (768, 288), (288, 768), (32000, 288),                 # config 1 (fp32 weights)
    (2048, 2048), (512, 2048), (256, 2048), (8192, 2048), (2048, 8192), (5632, 2048), (2048, 5632),
    (4096, 4096), (1024, 4096), (14336, 4096), (4096, 14336),        # config 5
    (1, 8), (3, 8), (5, 24), (7, 520), (2, 16384), (130, 1032),       # ragged tiles, tails
    (9, 20), (4, 7), (6, 2052), (3, 16392),                            # scalar fallback (d % 8, d > LDS)
]


@pytest.mark.parametrize("n,d", GEMV_SHAPES)
@pytest.mark.parametrize("fp16", [True, False])
def test_gemv_random(lib, n, d, fp16):
    if n * d > 40_000_000 and not fp16:
        pytest.skip("covered by the fp16 case")
    rng = np.random.default_rng(n * 7 + d)
    x = rng.standard_normal(d).astype(F)
    want = np.zeros(n, F)
    if fp16:
        w = (rng.standard_normal(n * d) * 0.02).astype(np.float16).view(np.uint16)
        orc.orc_matmul_f16w(want, x, w, n, d)
        wide = w.view(np.float16).astype(np.float64).reshape(n, d)
    else:
        w = (rng.standard_normal(n * d) * 0.02).astype(F)
        orc.orc_naive_matmul(want, x, w, n, d)
        wide = w.astype(np.float64).reshape(n, d)
    got = gemv_gpu(lib, x, w, n, d, capi.WEIGHT_FP16 if fp16 else capi.WEIGHT_FP32)
    exact = wide @ x.astype(np.float64)
    mag = np.abs(wide) @ np.abs(x.astype(np.float64))
    # fp32 accumulate: error bounded by a few eps of sum|w x| (pairwise tree)
    assert np.all(np.abs(got - exact) <= 16 * np.finfo(F).eps * mag + 1e-30)
    # and against the oracle (sequential fp32 sum), relative to the vector's scale
    assert np.max(np.abs(got - want)) <= 2e-3 * np.max(np.abs(want)) + 1e-30


def test_gemv_lm_head_full_size(lib):
    """128256 x 2048 binary16: the largest single launch of the decode step."""
    n, d = 128256, 2048
    w = capi.synth_normal_f16(n * d, 77, 0.02)
    x = np.random.default_rng(1).standard_normal(d).astype(F)
    got = gemv_gpu(lib, x, w, n, d, capi.WEIGHT_FP16)
    rows = np.random.default_rng(2).integers(0, n, 4000)
    wide = w.reshape(n, d)[rows].view(np.float16).astype(np.float64)
    exact = wide @ x.astype(np.float64)
    assert np.max(np.abs(got[rows] - exact)) < 2e-5 * np.max(np.abs(exact))
    # first / last rows and linearity: W.(2x) == 2 W.x exactly (power-of-two scale)
    assert abs(got[0] - float(w.reshape(n, d)[0].view(np.float16).astype(np.float64) @ x)) < 1e-4
    got2 = gemv_gpu(lib, (x * 2).astype(F), w, n, d, capi.WEIGHT_FP16)
    assert np.array_equal(bits(got2), bits(got * 2))


def test_gemv_edge_cases(lib):
    assert lib.lpp_gemv(None, None, None, None, 0, 16, capi.WEIGHT_FP16) == capi.LPP_OK  # empty
    x = DB.from_numpy(np.ones(8, F))
    assert lib.lpp_gemv(x.ptr, x.ptr, x.ptr, None, 1, 8, capi.WEIGHT_FP32) == capi.LPP_ERR_INVALID_ARG  # alias
    # misaligned weight pointer takes the scalar path and still agrees
    rng = np.random.default_rng(5)
    w = (rng.standard_normal(1 + 6 * 16) * 0.1).astype(np.float16).view(np.uint16)
    xv = rng.standard_normal(16).astype(F)
    dw, dx, dout = DB.from_numpy(w), DB.from_numpy(xv), DB(6 * 4)
    capi.check(lib.lpp_gemv(dout.ptr, dx.ptr, dw.at(2), None, 6, 16, capi.WEIGHT_FP16))
    want = w[1:].view(np.float16).astype(np.float64).reshape(6, 16) @ xv
    assert np.allclose(dout.to_numpy(F), want, rtol=1e-5, atol=1e-6)
    # precision values other than FP16 take the fp32 branch (matmul.cu:142-145)
    w32 = rng.standard_normal(4 * 8).astype(F)
    got = gemv_gpu(lib, np.ones(8, F), w32, 4, 8, 2)
    assert np.allclose(got, w32.reshape(4, 8).sum(1), rtol=1e-6)


def test_convert_f32_to_f16_bit_exact(lib):
    rng = np.random.default_rng(6)
    vals = np.concatenate([rng.standard_normal(100003).astype(F) * F(0.02),
                           rng.standard_normal(5000).astype(F) * F(1000),
                           (rng.standard_normal(5000) * 1e-6).astype(F),
                           np.array([0, -0.0, 65504, 65520, -65520, 1e-8, 2.9802322e-8, 6.1e-5], F),
                           np.arange(2048, 2100, dtype=F) + F(0.5)])
    src, dst = DB.from_numpy(vals), DB(vals.size * 2)
    capi.check(lib.lpp_convert_f32_to_f16(dst.ptr, src.ptr, vals.size))
    with np.errstate(over="ignore"):
        assert np.array_equal(dst.to_numpy(np.uint16), vals.astype(np.float16).view(np.uint16))
    assert lib.lpp_convert_f32_to_f16(None, None, 0) == capi.LPP_OK


# ---- rmsnorm / rope / swiglu / residual ---------------------------------------------

def test_rmsnorm_runtests_pattern_and_random(lib):  # runtests.cpp:471-520
    for n, xs in [(256, (0.5 + 0.1 * (np.arange(256) % 10)).astype(F)),
                  (288, np.random.default_rng(1).standard_normal(288).astype(F)),
                  (2048, np.random.default_rng(2).standard_normal(2048).astype(F) * 3),
                  (4096, np.random.default_rng(3).standard_normal(4096).astype(F) * 0.01),
                  (5, np.array([1, -2, 3, 0, 1e-3], F)), (1, np.array([2.0], F))]:
        g = np.ones(n, F) if n == 256 else (1 + 0.1 * np.random.default_rng(n).standard_normal(n)).astype(F)
        want = np.zeros(n, F)
        orc.orc_rmsnorm(want, xs, g, n)
        dx, dg, dout = DB.from_numpy(xs), DB.from_numpy(g), DB(n * 4)
        capi.check(lib.lpp_rmsnorm(dout.ptr, dx.ptr, dg.ptr, n))
        got = dout.to_numpy(F)
        # only the order of the sum of squares differs: a few ulp
        assert np.allclose(got, want, rtol=1e-6, atol=1e-12), n
        capi.check(lib.lpp_rmsnorm(dx.ptr, dx.ptr, dg.ptr, n))  # in place, model.cpp:357
        assert np.array_equal(bits(dx.to_numpy(F)), bits(got))


@pytest.mark.parametrize("dim,kv_dim,hs,pos,base", [
    (128, 128, 64, 5, 10000.0),        # runtests.cpp:522-579
    (288, 288, 48, 255, 10000.0),
    (2048, 512, 64, 511, 500000.0),
    (2048, 512, 64, 8447, 500000.0),
    (4096, 1024, 128, 1055, 500000.0),
    (16, 8, 2, 3, 10000.0),
    (64, 0, 8, 9, 10000.0),
])
def test_rope_bit_exact(lib, dim, kv_dim, hs, pos, base):
    """cos/sin come from the host C library, products are not contracted: the
    result equals the CPU operator bit for bit on the same machine."""
    if dim == 128:
        q = (1.0 + 0.1 * np.arange(dim)).astype(F)
        k = (0.5 + 0.1 * np.arange(dim)).astype(F)
    else:
        rng = np.random.default_rng(dim + pos)
        q, k = rng.standard_normal(dim).astype(F), rng.standard_normal(dim).astype(F)
    wq, wk = q.copy(), k.copy()
    orc.orc_rope(wq, wk, pos, dim, kv_dim, hs, base)
    dq, dk = DB.from_numpy(q), DB.from_numpy(k)
    capi.check(lib.lpp_rope(dq.ptr, dk.ptr if kv_dim else None, pos, dim, kv_dim, hs, base))
    assert np.array_equal(bits(dq.to_numpy(F)), bits(wq))
    assert np.array_equal(bits(dk.to_numpy(F)), bits(wk))


def test_swiglu(lib):  # runtests.cpp:581-630 plus tails the reference kernel drops
    for n in (256, 8192, 5632, 1, 3, 1027):
        if n == 256:
            h1 = (-2.0 + 0.02 * np.arange(n)).astype(F)
            h3 = (1.0 + 0.01 * np.arange(n)).astype(F)
        else:
            rng = np.random.default_rng(n)
            h1, h3 = (rng.standard_normal(n) * 4).astype(F), rng.standard_normal(n).astype(F)
        want = np.zeros(n, F)
        orc.orc_swiglu(want, h1, h3, n)
        d1, d3 = DB.from_numpy(h1), DB.from_numpy(h3)
        capi.check(lib.lpp_swiglu(d1.ptr, d1.ptr, d3.ptr, n))  # hb aliases h1, model.cpp:224
        got = d1.to_numpy(F)
        # expf on the device may differ from libm by an ulp or two
        assert np.allclose(got, want, rtol=1e-6, atol=1e-9), n


def test_residual_add_bit_exact(lib):  # runtests.cpp:750-797
    for n in (256, 2048, 1, 1023):
        a = (1.0 + 0.1 * np.arange(n)).astype(F) if n == 256 else np.random.default_rng(n).standard_normal(n).astype(F)
        b = (0.5 - 0.05 * np.arange(n)).astype(F) if n == 256 else np.random.default_rng(n + 1).standard_normal(n).astype(F)
        da, dbb = DB.from_numpy(a), DB.from_numpy(b)
        capi.check(lib.lpp_residual_add(da.ptr, da.ptr, dbb.ptr, n))  # out aliases a, model.cpp:218
        assert np.array_equal(bits(da.to_numpy(F)), bits(a + b))


# ---- KV scatter ------------------------------------------------------------------------

@pytest.mark.parametrize("L,nkv,hs,seq", [(3, 2, 4, 5), (2, 8, 64, 16), (2, 6, 48, 7), (1, 8, 128, 9)])
def test_scatter_kv_bit_exact(lib, L, nkv, hs, seq):
    """Every (layer, pos) written once; the whole cache must equal the layout of
    model.cpp:173 with values rounded to nearest-even binary16, and nothing else
    may be touched."""
    kv_dim = nkv * hs
    total = L * nkv * seq * hs
    rng = np.random.default_rng(L * 100 + hs)
    kc, vc = DB(total * 2), DB(total * 2)
    capi.check(lib.lpp_memset(kc.ptr, 0, total * 2))
    capi.check(lib.lpp_memset(vc.ptr, 0, total * 2))
    want_k = np.zeros((L, nkv, seq, hs), np.float16)
    want_v = np.zeros((L, nkv, seq, hs), np.float16)
    order = [(l, p) for l in range(L) for p in range(seq)]
    rng.shuffle(order)
    skip = set(order[:3])  # leave a few slots untouched
    for (l, p) in order:
        if (l, p) in skip:
            continue
        k = (rng.standard_normal(kv_dim) * 3).astype(F)
        v = (rng.standard_normal(kv_dim) * 1e-3).astype(F)
        dk, dv = DB.from_numpy(k), DB.from_numpy(v)
        capi.check(lib.lpp_scatter_kv(kc.ptr, vc.ptr, dk.ptr, dv.ptr, l, p, nkv, hs, seq))
        want_k[l, :, p, :] = k.reshape(nkv, hs).astype(np.float16)
        want_v[l, :, p, :] = v.reshape(nkv, hs).astype(np.float16)
    assert np.array_equal(kc.to_numpy(np.uint16), want_k.reshape(-1).view(np.uint16))
    assert np.array_equal(vc.to_numpy(np.uint16), want_v.reshape(-1).view(np.uint16))


def test_scatter_kv_large_offsets(lib):
    """Offsets beyond 2^31 bytes (config-5-sized caches) must not wrap."""
    L, nkv, hs, seq = 32, 8, 128, 4096  # 2^30 elements = 2 GiB per cache
    total = L * nkv * hs * seq
    kc = DB(total * 2)
    k = np.arange(nkv * hs, dtype=F)
    dk = DB.from_numpy(k)
    capi.check(lib.lpp_scatter_kv(kc.ptr, kc.ptr, dk.ptr, dk.ptr, L - 1, seq - 1, nkv, hs, seq))
    last_head_slot = ((L - 1) * nkv * seq + (nkv - 1) * seq + (seq - 1)) * hs
    got = kc.to_numpy(np.uint16, hs, byte_offset=last_head_slot * 2)
    assert np.array_equal(got, k[-hs:].astype(np.float16).view(np.uint16))


# ---- attention pieces ---------------------------------------------------------------------

@pytest.mark.parametrize("nh,nkv,hs,seq,pos,layer", [
    (4, 4, 16, 8, 7, 0), (32, 8, 64, 600, 511, 1), (32, 4, 64, 40, 16, 2), (6, 6, 48, 256, 255, 1),
    (32, 8, 128, 70, 64, 0), (8, 2, 8, 20, 0, 1), (4, 2, 12, 9, 8, 0),
])
def test_multihead_gemv(lib, nh, nkv, hs, seq, pos, layer):
    L = layer + 1
    rng = np.random.default_rng(nh * 31 + pos)
    kc16 = rng.standard_normal((L, nkv, seq, hs)).astype(np.float16)
    q = rng.standard_normal(nh * hs).astype(F)
    dk, dq, dout = DB.from_numpy(kc16.view(np.uint16)), DB.from_numpy(q), DB(nh * seq * 4)
    capi.check(lib.lpp_memset(dout.ptr, 0xFF, nh * seq * 4))
    capi.check(lib.lpp_multihead_gemv(dout.ptr, dq.ptr, dk.ptr, layer, pos, nh, nkv, hs, seq))
    got = dout.to_numpy(F).reshape(nh, seq)
    g = nh // nkv
    for h in range(nh):
        kh = kc16[layer, h // g, :pos + 1].astype(F)
        want = np.zeros(pos + 1, F)
        orc.orc_naive_matmul(want, q[h * hs:(h + 1) * hs].copy(), kh.reshape(-1), pos + 1, hs)  # model.cpp:186
        mag = np.abs(kh.astype(np.float64)) @ np.abs(q[h * hs:(h + 1) * hs].astype(np.float64))
        assert np.all(np.abs(got[h, :pos + 1] - want) <= 8 * np.finfo(F).eps * mag + 1e-30)
    # entries beyond pos are not written
    assert np.all(dout.to_numpy(np.uint32).reshape(nh, seq)[:, pos + 1:] == 0xFFFFFFFF)


def test_scale_multihead_bit_exact(lib):  # runtests.cpp:696-748
    nh, n, stride = 4, 32, 64
    att = np.zeros((nh, stride), F)
    att[:, :] = 1.0 + 0.1 * np.arange(stride)
    d = DB.from_numpy(att)
    capi.check(lib.lpp_scale_multihead(d.ptr, 0.125, nh, n, stride))
    got = d.to_numpy(F).reshape(nh, stride)
    assert np.array_equal(bits(got[:, :n]), bits(att[:, :n] * F(0.125)))
    assert np.array_equal(bits(got[:, n:]), bits(att[:, n:]))


# (rows of up to 1024, 4096 and 16384 values take a kernel that keeps them in registers, longer ones the general kernel)
@pytest.mark.parametrize("nh,n,stride", [(4, 32, 64), (32, 512, 2048), (32, 8448, 16384), (6, 1, 256), (3, 1025, 1030),
                                         (2, 1024, 1024), (2, 4096, 4100), (2, 4097, 4100), (2, 16384, 16384),
                                         (2, 16385, 16400), (1, 40000, 40000)])
def test_softmax_multihead(lib, nh, n, stride):  # runtests.cpp:633-694
    if (nh, n, stride) == (4, 32, 64):
        x = np.zeros((nh, stride), F)
        for h in range(nh):
            x[h, :] = -5.0 + 0.3 * np.arange(stride) + h
    else:
        x = (np.random.default_rng(n).standard_normal((nh, stride)) * 4).astype(F)
    d = DB.from_numpy(x)
    capi.check(lib.lpp_softmax_multihead(d.ptr, d.ptr, nh, n, stride))  # in place, model.cpp:153
    got = d.to_numpy(F).reshape(nh, stride)
    for h in range(nh):
        want = x[h, :n].copy()
        orc.orc_softmax(want, n)
        exact = np.exp(x[h, :n].astype(np.float64) - float(x[h, :n].max()))
        exact /= exact.sum()
        # tree sum on the device: a few ulp from the exact value ...
        assert np.allclose(got[h, :n], exact, rtol=3e-6, atol=1e-12)
        # ... while the CPU's running fp32 sum drifts by up to ~n ulp; still far inside 2e-3
        assert np.allclose(got[h, :n], want, rtol=1e-4, atol=1e-12)
        assert abs(got[h, :n].astype(np.float64).sum() - 1) < 1e-5
    assert np.array_equal(bits(got[:, n:]), bits(x[:, n:]))


@pytest.mark.parametrize("nh,gqa,hs,seq,n", [
    (4, 1, 16, 8, 8),           # runtests.cpp:799-875 shape
    (32, 4, 64, 600, 512), (32, 8, 64, 64, 17), (6, 1, 48, 256, 256), (32, 4, 128, 1100, 1056), (8, 4, 8, 10, 1),
    (4, 2, 12, 9, 9),
    # long contexts: several workgroups per head, partial sums combined by the last to finish
    (32, 4, 64, 16384, 8193), (8, 1, 128, 4200, 4099), (200, 4, 32, 1024, 1000),
])
def test_aggregation_multihead(lib, nh, gqa, hs, seq, n):
    nkv = nh // gqa
    rng = np.random.default_rng(nh + n)
    if seq == 8 and hs == 16:
        v16 = (0.1 * (np.arange(nkv * seq * hs) % 10)).astype(np.float16).reshape(nkv, seq, hs)
        att = np.full((nh, seq), 1.0 / 8, F)
    else:
        v16 = rng.standard_normal((nkv, seq, hs)).astype(np.float16)
        att = rng.random((nh, seq)).astype(F)
        att /= att[:, :n].sum(1, keepdims=True)
    gpu_v = v16.view(np.uint16).copy()
    gpu_v[:, n:, :] = 0x7e00  # what lies past the context is never read into a sum: NaN there must not show
    dv, da, dout = DB.from_numpy(gpu_v), DB.from_numpy(att), DB(nh * hs * 4)
    capi.check(lib.lpp_aggregation_multihead(dout.ptr, dv.ptr, da.ptr, nh, n, hs, gqa, seq))
    got = dout.to_numpy(F).reshape(nh, hs)
    # a second launch right behind the first gives the same bits (fixed summation order, scratch left clean)
    capi.check(lib.lpp_aggregation_multihead(dout.ptr, dv.ptr, da.ptr, nh, n, hs, gqa, seq))
    assert np.array_equal(bits(dout.to_numpy(F).reshape(nh, hs)), bits(got))
    for h in range(nh):
        vh = v16[h // gqa, :n].astype(np.float64)
        exact = att[h, :n].astype(np.float64) @ vh
        mag = att[h, :n].astype(np.float64) @ np.abs(vh)
        assert np.all(np.abs(got[h] - exact) <= 16 * np.finfo(F).eps * mag + 1e-30)
        # the reference's bar: 1 % relative + 1e-4 (runtests.cpp:858)
        assert np.all(np.abs(got[h] - exact) <= 0.01 * np.abs(exact) + 1e-4)


# ---- sampler -----------------------------------------------------------------------------------

def sample_gpu(lib, logits, temperature, penalty, history, r, topp=0.9):
    dl = DB.from_numpy(np.ascontiguousarray(logits, F))
    dtok = DB(4)
    if history is not None and len(history) > 0:
        dh = DB.from_numpy(np.asarray(history, np.int32))
        hp, hl = dh.ptr, len(history)
    else:
        hp, hl = None, 0
    capi.check(lib.lpp_sample(dl.ptr, len(logits), temperature, topp, penalty, hp, hl, dtok.ptr, None, r))
    return int(dtok.to_numpy(np.int32)[0]), dl.to_numpy(F)


@pytest.mark.parametrize("vocab", [97, 1000, 32000, 128256, 262145])
def test_sample_greedy_index_exact(lib, vocab):
    rng = np.random.default_rng(vocab)
    lg = rng.standard_normal(vocab).astype(F)
    hi = lg.max() + F(1)
    ties = sorted(rng.choice(vocab, 3, replace=False).tolist())
    for t in ties:
        lg[t] = hi  # equal maxima: the lowest index must win (model.cpp:275-281)
    hist = [ties[0], ties[0], 5, -1, vocab + 3, ties[2]]
    for pen, history in [(1.0, None), (1.0, hist), (1.3, hist), (1.3, None)]:
        want, after = ob.orc_sample(lg, 0.0, 1.0, pen, history, 0.0)
        got, gafter = sample_gpu(lib, lg, 0.0, pen, history, 0.0)
        assert got == want
        assert np.array_equal(bits(gafter), bits(after))  # penalised logits, bit-exact


def test_sample_penalty_per_occurrence_bit_exact(lib):
    vocab = 5000
    rng = np.random.default_rng(3)
    lg = (rng.standard_normal(vocab) * 3).astype(F)
    lg[7] = 0.0
    hist = rng.integers(0, 40, 64).tolist() + [7, 7, -5, vocab, vocab + 1]  # many repeats, zero logit, bad ids
    want, after = ob.orc_sample(lg, 0.0, 1.0, 1.1, hist, 0.0)
    got, gafter = sample_gpu(lib, lg, 0.0, 1.1, hist, 0.0)
    assert got == want and np.array_equal(bits(gafter), bits(after))
    long_hist = rng.integers(0, vocab, 3000).tolist()  # window longer than one workgroup pass
    want, after = ob.orc_sample(lg, 0.0, 1.0, 1.05, long_hist, 0.0)
    got, gafter = sample_gpu(lib, lg, 0.0, 1.05, long_hist, 0.0)
    assert got == want and np.array_equal(bits(gafter), bits(after))


@pytest.mark.parametrize("vocab,temp,pen", [(97, 1.0, 1.0), (32000, 0.8, 1.1), (128256, 0.8, 1.1), (128256, 1.5, 1.0)])
def test_sample_categorical(lib, vocab, temp, pen):
    """Token identity against the oracle for many draws.  A different token is
    accepted only if r sits within 1e-4 of a bucket edge of the oracle's CDF (the
    parallel scan rounds differently from the CPU's running sum); the logits bar
    of 2e-3 would allow far more."""
    rng = np.random.default_rng(vocab + int(temp * 10))
    lg = (rng.standard_normal(vocab) * 2.5).astype(F)
    hist = rng.integers(0, vocab, 64).tolist()
    hist[10] = hist[11] = hist[12]
    draws = np.concatenate([capi.synth_uniform_f32(60, vocab), np.array([0.0, 1.0, 0.99999994, 1e-7, 0.5], F)])
    _, want_probs = ob.orc_sample(lg, temp, 1.0, pen, hist, 0.5)
    # the exact CDF (fp64) of the penalised, tempered logits: the device's token must sit where
    # the draw falls in it, to within the rounding of an fp32 sum over the vocabulary
    z = ob.orc_sample(lg, 0.0, 1.0, pen, hist, 0.0)[1].astype(np.float64) / temp
    p64 = np.exp(z - z.max())
    c64 = np.cumsum(p64 / p64.sum())
    near = 0
    for r in draws:
        want, lo, hi = ob.orc_sample_cdf(lg, temp, pen, hist, float(r))
        got, probs = sample_gpu(lib, lg, temp, pen, hist, float(r))
        below = c64[got - 1] if got > 0 else 0.0
        assert below - 2e-6 <= float(r) < c64[got] + 2e-6 or got == vocab - 1, (float(r), got, below, c64[got])
        if got != want:
            near += 1
            assert min(abs(float(r) - lo), abs(float(r) - hi)) < 1e-4, (float(r), want, got, lo, hi)
    # With 128256 buckets of ~8e-6 each, the drift of the CPU's running fp32 sum (up to ~1e-5 by the
    # end of the vocabulary) moves a fair share of draws into a neighbouring bucket; with few
    # buckets it must not happen more than occasionally.
    assert near <= (3 if vocab < 50000 else len(draws) // 2)
    # the buffer is left holding probabilities, as on the CPU (model.cpp:290)
    # (the CPU's running fp32 sum over the vocabulary drifts by up to ~n ulp, the
    # device's tree sum does not: compare loosely with the oracle, tightly with fp64)
    assert np.allclose(probs, want_probs, rtol=3e-4, atol=1e-12)
    pen_lg = ob.orc_sample(lg, 0.0, 1.0, pen, hist, 0.0)[1].astype(np.float64)  # penalised logits, exact
    scaled = (pen_lg.astype(F) / F(temp)).astype(np.float64)
    exact = np.exp(scaled - scaled.max())
    exact /= exact.sum()
    assert np.allclose(probs, exact, rtol=4e-6, atol=1e-12)
    assert abs(probs.astype(np.float64).sum() - 1) < 1e-5


def test_sample_r_at_or_above_total_mass(lib):
    lg = np.log(np.array([0.1, 0.2, 0.3, 0.4], F))
    assert sample_gpu(lib, lg, 1.0, 1.0, None, 1.0)[0] == 3   # model.cpp:302 fallback
    assert sample_gpu(lib, lg, 1.0, 1.0, None, 0.0)[0] == 0
    assert sample_gpu(lib, lg, 1.0, 1.0, None, 0.35)[0] == 2
    two = np.zeros(2, F)
    assert sample_gpu(lib, two, 1.0, 1.0, None, 0.5)[0] == 1  # strict <
    assert sample_gpu(lib, two, 1.0, 1.0, None, float(np.nextafter(F(0.5), F(0))))[0] == 0
    assert sample_gpu(lib, np.array([3.0], F), 0.7, 1.0, None, 0.3)[0] == 0  # vocab of one
