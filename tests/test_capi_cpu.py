"""CPU-side checks of the C ABI: the library loads without a GPU, exports every
symbol include/lpp.h declares, rejects bad arguments with a status instead of
aborting, and its host-side helpers (synthetic tensors, binary16 conversion)
are deterministic and exact.  No kernel is launched here."""
import ctypes as C
import re
from pathlib import Path

import numpy as np
import pytest

from lighterpp_amd import CONFIGS, Shape, capi, synth_tensor

ROOT = Path(__file__).resolve().parent.parent
F = np.float32


def declared_symbols():
    text = (ROOT / "include" / "lpp.h").read_text()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(lpp_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    lib = capi.load()
    names = declared_symbols()
    assert len(names) >= 45
    for n in names:
        assert hasattr(lib, n), f"{n} declared in include/lpp.h but not exported"
    assert set(names) == set(capi.SIGNATURES), "binding table and header disagree"


def test_compat_header_covers_the_twelve_wrappers():
    """include/lpp_kernels_compat.h must offer every host wrapper of the reference's
    kernels.cuh:24-36 under its original name."""
    text = (ROOT / "include" / "lpp_kernels_compat.h").read_text()
    for name in ["cuda_convert_f32_to_f16", "cuda_gemv", "cuda_rmsnorm", "cuda_rope", "cuda_swiglu",
                 "cuda_softmax_multihead", "cuda_scale_multihead", "cuda_aggregation_multihead",
                 "cuda_residual_add", "cuda_scatter_kv", "cuda_multihead_gemv", "cuda_sample"]:
        assert re.search(rf"\b{name}\s*\(", text), name
    assert "MAX_SHARED_FLOATS" in text and "checkCuda" in text


def test_compat_header_compiles_and_links_as_cxx(tmp_path):
    """A translation unit written against the reference's kernels.cuh surface must
    compile with plain g++ against the compat header and link with the library."""
    import shutil
    import subprocess
    if shutil.which("g++") is None:
        pytest.skip("g++ not available")
    src = tmp_path / "caller.cpp"
    src.write_text(
        "enum WeightPrecision : int { WEIGHT_FP32 = 0, WEIGHT_FP16 = 1, WEIGHT_INT4 = 2 };\n"
        '#include "lpp_kernels_compat.h"\n'
        "int main() {\n"
        "  float* f = nullptr; __half* h = nullptr; int* i = nullptr;\n"
        "  if (MAX_SHARED_FLOATS < 14336) return 1;\n"
        "  if (false) {\n"
        "    cuda_convert_f32_to_f16(h, f, 0); cuda_gemv(f, f, h, h, 0, 0, WEIGHT_FP16); cuda_rmsnorm(f, f, f, 0);\n"
        "    cuda_rope(f, f, 0, 0, 0, 0, 1.f); cuda_swiglu(f, f, f, 0); cuda_softmax_multihead(f, f, 0, 0, 0);\n"
        "    cuda_scale_multihead(f, 1.f, 0, 0, 0); cuda_aggregation_multihead(f, h, f, 0, 0, 0, 0, 0);\n"
        "    cuda_residual_add(f, f, f, 0); cuda_scatter_kv(h, h, f, f, 0, 0, 0, 0, 0);\n"
        "    cuda_multihead_gemv(f, f, h, 0, 0, 0, 0, 0, 0); cuda_sample(f, 0, 0.f, 0.f, 0.f, i, 0, i, nullptr);\n"
        "  }\n"
        "  cuda_gemv(nullptr, nullptr, nullptr, nullptr, 0, 0, WEIGHT_FP16);  // n == 0: accepted, no launch\n"
        "  return 0;\n"
        "}\n")
    exe = tmp_path / "caller"
    libdir = ROOT / "lighterpp_amd"
    subprocess.run(["g++", "-std=c++17", "-Wall", "-Wextra", "-Werror", f"-I{ROOT / 'include'}", str(src),
                    f"-L{libdir}", "-llpp_hip", f"-Wl,-rpath,{libdir}", "-o", str(exe)], check=True)
    assert subprocess.run([str(exe)]).returncode == 0


def test_version_and_error_string():
    lib = capi.load()
    assert b"gfx950" in lib.lpp_version()
    # Argument validation happens before any device work.
    st = lib.lpp_gemv(None, None, None, None, 4, 4, capi.WEIGHT_FP16)
    assert st == capi.LPP_ERR_INVALID_ARG
    assert b"lpp_gemv" in lib.lpp_last_error()
    assert lib.lpp_rope(None, None, 0, 8, 8, 4, 10000.0) == capi.LPP_ERR_INVALID_ARG
    assert lib.lpp_scatter_kv(1, 1, 1, 1, 0, 5, 2, 4, 5) == capi.LPP_ERR_INVALID_ARG  # pos == seq_len
    assert lib.lpp_sample(None, 10, 0.0, 1.0, 1.0, None, 0, None, None, 0.0) == capi.LPP_ERR_INVALID_ARG
    bad = capi.LppConfig(64, 128, 1, 6, 4, 10, 8, 10000.0, capi.WEIGHT_FP16)  # 64 % 6 != 0
    h = C.c_void_p()
    assert lib.lpp_model_create(C.byref(h), C.byref(bad)) == capi.LPP_ERR_INVALID_ARG
    assert not h.value


def test_synth_is_deterministic_and_sliceable():
    a = capi.synth_normal_f32(10000, 42, 0.02)
    b = capi.synth_normal_f32(10000, 42, 0.02)
    assert np.array_equal(a, b)
    part = capi.synth_normal_f32(100, 42, 0.02, first_index=5000)
    assert np.array_equal(part, a[5000:5100])
    assert not np.array_equal(a, capi.synth_normal_f32(10000, 43, 0.02))
    big = capi.synth_normal_f32(400000, 7, 0.02)
    assert abs(big.mean()) < 2e-4 and abs(big.std() - 0.02) < 2e-4
    # tails of a normal, not a clipped or uniform imitation
    assert 0.0015 < np.mean(np.abs(big) > 0.06) < 0.0040
    u = capi.synth_uniform_f32(100000, 3)
    assert u.min() >= 0 and u.max() < 1 and abs(u.mean() - 0.5) < 0.01
    ids = capi.synth_token_ids(1000, 9, 128256)
    assert ids.min() >= 0 and ids.max() < 128256 and len(set(ids.tolist())) > 900


def test_synth_f16_is_rounded_f32():
    a = capi.synth_normal_f32(5000, 11, 0.02)
    h = capi.synth_normal_f16(5000, 11, 0.02)
    assert np.array_equal(h, a.astype(np.float16).view(np.uint16))


def test_host_half_conversions_exact():
    bits = np.arange(65536, dtype=np.uint16)
    wide = capi.f16_to_f32(bits)
    want = bits.view(np.float16).astype(F)
    ok = ~np.isnan(want)
    assert np.array_equal(wide[ok].view(np.uint32), want[ok].view(np.uint32))
    assert np.array_equal(np.isnan(wide), ~ok)
    back = capi.f32_to_f16(wide[ok])
    assert np.array_equal(back, bits[ok])
    rng = np.random.default_rng(0)
    vals = np.concatenate([rng.standard_normal(50000).astype(F) * F(0.02), rng.standard_normal(5000).astype(F) * F(1e3),
                           (rng.standard_normal(5000) * 1e-6).astype(F)])
    with np.errstate(over="ignore"):
        assert np.array_equal(capi.f32_to_f16(vals), vals.astype(np.float16).view(np.uint16))


def test_synth_tensor_recipe():
    shape = Shape(64, 160, 3, 8, 2, 320, 32, 10000.0, fp16=True, tied=True)
    emb = synth_tensor(shape, capi.T_TOKEN_EMBEDDING, 5)
    cls = synth_tensor(shape, capi.T_WCLS, 5)
    assert emb.dtype == F and cls.dtype == np.uint16 and emb.shape == (320, 64)
    assert np.array_equal(capi.f16_to_f32(cls), emb)  # tied: same binary16 values
    assert np.all(synth_tensor(shape, capi.T_RMS_FFN, 5) == 1)
    assert synth_tensor(shape, capi.T_W1, 5).shape == (3, 160, 64)


def test_bytes_per_token_matches_published_plan():
    """Average algorithmic bytes/token of the benchmark windows (the figures the
    roofline fraction is computed from)."""
    def avg(shape, first, n):
        return np.mean([shape.bytes_per_token(p) for p in range(first, first + n)]) / 1e9
    assert abs(avg(CONFIGS["c1_llama2c_15m_fp32"], 8, 256) - 0.0617) < 2e-4
    assert abs(avg(CONFIGS["c2_tinyllama_1b_fp16"], 16, 512) - 2.0754) < 2e-3
    assert abs(avg(CONFIGS["c3_llama32_1b_fp16"], 0, 512) - 2.4802) < 2e-3
    assert abs(avg(CONFIGS["c4_llama32_1b_longctx_fp16"], 8192, 256) - 2.7445) < 2e-3
    assert abs(avg(CONFIGS["c5_llama3_8b_fp16"], 32, 1024) - 15.082) < 2e-2
    assert CONFIGS["c3_llama32_1b_fp16"].matrix_params() == 1_235_746_816 or \
        abs(CONFIGS["c3_llama32_1b_fp16"].matrix_params() / 1e6 - 1235.7) < 0.1
