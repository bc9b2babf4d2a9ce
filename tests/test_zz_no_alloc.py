"""lpp_prefill_gemm_noalloc (include/lpp.h): the prefill's GEMM with its binary16
head / remainder scratch in the library's device image instead of two allocations.
It must give lpp_prefill_gemm's result bit for bit (same kernels, same order), on two
calls in a row, the second smaller than the first so that it runs over what the first
left in the shared scratch; sizes beyond the built-in scratch are rejected."""
import numpy as np
import pytest

from lighterpp_amd import capi
from lighterpp_amd.capi import DeviceBuffer as DB

pytestmark = pytest.mark.gpu
F = np.float32


def _case(lib, seed, n, k, t, accumulate):
    rng = np.random.default_rng(seed)
    w = (rng.standard_normal((n, k)) * 0.05).astype(np.float16)
    x = (rng.standard_normal((t, k)) * 3.0).astype(F)
    x[1, :] = 1.0 / 3.0  # needs the remainder term
    y0 = rng.standard_normal((t, n)).astype(F)
    dw, dx = DB.from_numpy(w), DB.from_numpy(x)
    d_ref, d_new = DB.from_numpy(y0), DB.from_numpy(y0)
    capi.check(lib.lpp_prefill_gemm(d_ref.ptr, dw.ptr, dx.ptr, n, k, t, accumulate))
    capi.check(lib.lpp_prefill_gemm_noalloc(d_new.ptr, dw.ptr, dx.ptr, n, k, t, accumulate))
    capi.check(lib.lpp_synchronize())
    want = d_ref.to_numpy(F, t * n)
    got = d_new.to_numpy(F, t * n)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32)), \
        f"n {n} k {k} t {t}: {np.count_nonzero(got != want)} of {got.size} outputs differ"
    f64 = x.astype(np.float64) @ w.astype(np.float64).T + (y0 if accumulate else 0.0)
    assert np.max(np.abs(got.reshape(t, n) - f64)) <= 1e-5 * np.max(np.abs(f64))


def test_noalloc_gemm_matches_allocating_gemm_twice_in_a_row():
    lib = capi.load()
    capi.check(lib.lpp_init(0))
    print("no-alloc GEMM: n 256 k 4096 t 512 (fills the scratch), then n 384 k 1024 t 128", flush=True)
    _case(lib, 11, 256, 4096, 512, 0)   # 2097152 elements: the whole scratch
    _case(lib, 12, 384, 1024, 128, 1)   # smaller, over the first call's leftovers
    _case(lib, 13, 128, 32, 128, 0)     # smallest shape the GEMM takes


def _free_device_bytes():
    """hipMemGetInfo of the HIP runtime the library itself is linked against."""
    import ctypes as C
    hip = C.CDLL("libamdhip64.so")
    free, total = C.c_size_t(0), C.c_size_t(0)
    assert hip.hipMemGetInfo(C.byref(free), C.byref(total)) == 0
    return free.value


def test_noalloc_gemm_allocates_nothing_and_queues_without_a_sync():
    """What the entry point is for: device memory in use does not move across its calls (nothing allocated, nothing
    freed), and two calls of different shapes queued back to back, with no synchronisation between them, both give
    the allocating entry point's bits (the second overwrites the scratch the first is still being read from only
    after it: one stream)."""
    lib = capi.load()
    capi.check(lib.lpp_init(0))
    rng = np.random.default_rng(21)
    cases = []
    for n, k, t, acc in [(256, 2048, 256, 0), (128, 512, 128, 1)]:
        w = (rng.standard_normal((n, k)) * 0.05).astype(np.float16)
        x = (rng.standard_normal((t, k)) * 3.0).astype(F)
        y0 = rng.standard_normal((t, n)).astype(F)
        dw, dx = DB.from_numpy(w), DB.from_numpy(x)
        d_ref, d_new = DB.from_numpy(y0), DB.from_numpy(y0)
        capi.check(lib.lpp_prefill_gemm(d_ref.ptr, dw.ptr, dx.ptr, n, k, t, acc))
        cases.append((n, k, t, acc, dw, dx, d_ref, d_new))
    capi.check(lib.lpp_synchronize())
    before = _free_device_bytes()
    for n, k, t, acc, dw, dx, d_ref, d_new in cases:  # queued one behind the other
        capi.check(lib.lpp_prefill_gemm_noalloc(d_new.ptr, dw.ptr, dx.ptr, n, k, t, acc))
    after_queue = _free_device_bytes()
    capi.check(lib.lpp_synchronize())
    after = _free_device_bytes()
    assert before == after_queue == after, (before, after_queue, after)
    for n, k, t, acc, dw, dx, d_ref, d_new in cases:
        want, got = d_ref.to_numpy(F, t * n), d_new.to_numpy(F, t * n)
        assert np.array_equal(got.view(np.uint32), want.view(np.uint32)), (n, k, t)


def test_noalloc_gemm_rejects_what_does_not_fit():
    lib = capi.load()
    capi.check(lib.lpp_init(0))
    d = DB(1 << 20)
    assert lib.lpp_prefill_gemm_noalloc(d.ptr, d.ptr, d.ptr, 128, 8192, 512, 0) == capi.LPP_ERR_INVALID_ARG
    assert b"scratch" in lib.lpp_last_error()
    for n, k, t in [(100, 32, 128), (128, 48, 128), (128, 32, 100), (128, 32, 0)]:
        assert lib.lpp_prefill_gemm_noalloc(d.ptr, d.ptr, d.ptr, n, k, t, 0) == capi.LPP_ERR_INVALID_ARG
