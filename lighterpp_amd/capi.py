"""ctypes view of liblpp_hip.so (the C ABI declared in include/lpp.h).

This module is plumbing for the tests and the benchmark; the product is the
shared library.  It fails loudly when the library has not been built: there is
no CPU fallback behind any of these calls.
"""
from __future__ import annotations

import ctypes as C
import os
from pathlib import Path

import numpy as np

PKG_DIR = Path(__file__).resolve().parent
LIB_PATH = PKG_DIR / "liblpp_hip.so"

# ---- constants of include/lpp.h ------------------------------------------------
LPP_OK = 0
LPP_ERR_INVALID_ARG = 1
LPP_ERR_HIP = 2
LPP_ERR_OOM = 3
LPP_ERR_STATE = 4
LPP_ERR_UNSUPPORTED = 5

WEIGHT_FP32, WEIGHT_FP16, WEIGHT_INT4 = 0, 1, 2

(T_TOKEN_EMBEDDING, T_RMS_ATT, T_WQ, T_WK, T_WV, T_WO, T_RMS_FFN, T_W1, T_W2, T_W3,
 T_RMS_FINAL, T_WCLS) = range(12)
TENSOR_NAMES = ["token_embedding", "rms_att", "wq", "wk", "wv", "wo", "rms_ffn", "w1", "w2", "w3",
                "rms_final", "wcls"]

(B_X, B_XB, B_XB2, B_HB, B_HE, B_Q, B_K, B_V, B_ATT, B_LOGITS, B_KEY_CACHE, B_VALUE_CACHE) = range(12)

PATH_OPS, PATH_FUSED, PATH_PERSISTENT = 0, 1, 2
GGML_F32, GGML_F16 = 0, 1
PREFILL_EXACT, PREFILL_FAST = 0, 1
# enum lpp_test_option
(OPT_DECODE_XCD_HANDOVERS, OPT_DECODE_XCD_QKV, OPT_DECODE_PARKING, OPT_DECODE_LANE_ITEM, OPT_DECODE_FAIL_TICKETS,
 OPT_DECODE_XCD_ATTENTION, OPT_PREFILL_STAGED_GEMM, OPT_PREFILL_WIDE_TILES, OPT_PREFILL_FUSED_FFN,
 OPT_PREFILL_MFMA_ATTENTION, OPT_DECODE_CALIBRATE, OPT_COUNT) = range(12)
OPT_DEFAULTS = {OPT_DECODE_XCD_HANDOVERS: 1, OPT_DECODE_XCD_QKV: 1, OPT_DECODE_PARKING: 1, OPT_DECODE_LANE_ITEM: 1,
                OPT_DECODE_FAIL_TICKETS: 0, OPT_DECODE_XCD_ATTENTION: 1, OPT_PREFILL_STAGED_GEMM: 1,
                OPT_PREFILL_WIDE_TILES: 1, OPT_PREFILL_FUSED_FFN: 1, OPT_PREFILL_MFMA_ATTENTION: 1, OPT_DECODE_CALIBRATE: 1}
TOKENIZER_SENTENCEPIECE, TOKENIZER_BPE = 0, 1


class LppConfig(C.Structure):
    """Config of src/model.h:21-31."""
    _fields_ = [("dim", C.c_int), ("hidden_dim", C.c_int), ("n_layers", C.c_int), ("n_heads", C.c_int),
                ("n_kv_heads", C.c_int), ("vocab_size", C.c_int), ("seq_len", C.c_int),
                ("rope_base", C.c_float), ("weight_precision", C.c_int)]


class LppGenStats(C.Structure):
    _fields_ = [("wall_seconds", C.c_double), ("device_ms", C.c_double), ("kernel_ms_sum", C.c_double),
                ("kernel_launches", C.c_int), ("tokens", C.c_int)]


class LppRunResult(C.Structure):
    """lpp_run_result: what the driver loop of src/main.cpp:139-232 leaves behind."""
    _fields_ = [("n_tokens", C.c_int), ("final_pos", C.c_int), ("stopped_by_eos", C.c_int),
                ("reported_count", C.c_int), ("history_len", C.c_int), ("history", C.c_int * 64),
                ("wall_seconds", C.c_double)]


class LppKernelTime(C.Structure):
    _fields_ = [("name", C.c_char * 32), ("launches_per_token", C.c_int), ("avg_ms", C.c_double),
                ("bytes_per_launch", C.c_double)]


class LppError(RuntimeError):
    def __init__(self, status: int, message: str):
        super().__init__(f"lpp status {status}: {message}")
        self.status = status


# Every symbol include/lpp.h declares: name -> (restype, argtypes).
_vp, _i, _f, _sz, _u64 = C.c_void_p, C.c_int, C.c_float, C.c_size_t, C.c_uint64
_ip = C.POINTER(C.c_int)
SIGNATURES = {
    # A. operators
    "lpp_convert_f32_to_f16": (_i, [_vp, _vp, _i]),
    "lpp_gemv": (_i, [_vp, _vp, _vp, _vp, _i, _i, _i]),
    "lpp_rmsnorm": (_i, [_vp, _vp, _vp, _i]),
    "lpp_rope": (_i, [_vp, _vp, _i, _i, _i, _i, _f]),
    "lpp_swiglu": (_i, [_vp, _vp, _vp, _i]),
    "lpp_softmax_multihead": (_i, [_vp, _vp, _i, _i, _i]),
    "lpp_scale_multihead": (_i, [_vp, _f, _i, _i, _i]),
    "lpp_aggregation_multihead": (_i, [_vp, _vp, _vp, _i, _i, _i, _i, _i]),
    "lpp_residual_add": (_i, [_vp, _vp, _vp, _i]),
    "lpp_scatter_kv": (_i, [_vp, _vp, _vp, _vp, _i, _i, _i, _i, _i]),
    "lpp_multihead_gemv": (_i, [_vp, _vp, _vp, _i, _i, _i, _i, _i, _i]),
    "lpp_sample": (_i, [_vp, _i, _f, _f, _f, _vp, _i, _vp, _vp, _f]),
    # B. model
    "lpp_model_create": (_i, [C.POINTER(_vp), C.POINTER(LppConfig)]),
    "lpp_model_destroy": (_i, [_vp]),
    "lpp_model_tensor_bytes": (_i, [_vp, _i, C.POINTER(_sz)]),
    "lpp_model_upload": (_i, [_vp, _i, _sz, _vp, _sz]),
    "lpp_model_tie_classifier": (_i, [_vp]),
    "lpp_model_tensor_ptr": (_i, [_vp, _i, C.POINTER(_vp)]),
    "lpp_model_buffer_ptr": (_i, [_vp, _i, C.POINTER(_vp), C.POINTER(_sz)]),
    "lpp_model_set_path": (_i, [_vp, _i]),
    "lpp_model_set_spin_limit": (_i, [_vp, C.c_uint]),
    "lpp_model_set_sequence_base": (_i, [_vp, C.c_uint]),
    "lpp_model_reset": (_i, [_vp]),
    "lpp_attention": (_i, [_vp, _i, _i]),
    "lpp_transformer_block": (_i, [_vp, _i, _i]),
    "lpp_forward": (_i, [_vp, _i, _i, _f, _f, _f, _vp, _i, _f, _ip]),
    "lpp_generate": (_i, [_vp, _i, _i, _i, _f, _f, _f, _vp, _ip, _i, _vp, _vp, C.POINTER(LppGenStats)]),
    "lpp_profile_kernels": (_i, [_vp, _i, _i, C.POINTER(LppKernelTime), _i, _ip]),
    "lpp_trace_token": (_i, [_vp, _i, C.POINTER(C.c_ulonglong), _i, _ip, _ip]),
    "lpp_trace_token_all": (_i, [_vp, _i, _vp, _i, _ip, _ip, _ip]),
    # D. checkpoint reader and driver loop
    "lpp_checkpoint_open": (_i, [C.POINTER(_vp), C.c_char_p]),
    "lpp_checkpoint_close": (_i, [_vp]),
    "lpp_checkpoint_config": (_i, [_vp, C.POINTER(LppConfig)]),
    "lpp_checkpoint_tensor": (_i, [_vp, _i, C.POINTER(_vp), C.POINTER(_sz)]),
    "lpp_model_load_checkpoint": (_i, [C.POINTER(_vp), _vp]),
    "lpp_run": (_i, [_vp, _vp, _i, _i, _f, _f, _vp, _vp, _i, C.POINTER(LppRunResult)]),
    "lpp_run_batched_prefill": (_i, [_vp, _vp, _i, _i, _f, _f, _vp, _vp, _i, C.POINTER(LppRunResult)]),
    "lpp_prefill_supported": (_i, [_vp]),
    "lpp_model_set_prefill_mode": (_i, [_vp, _i]),
    "lpp_prefill": (_i, [_vp, _vp, _i, _i]),
    "lpp_prefill_gemm": (_i, [_vp, _vp, _vp, _i, _i, _i, _i]),
    "lpp_prefill_gemm_noalloc": (_i, [_vp, _vp, _vp, _i, _i, _i, _i]),
    "lpp_gguf_open": (_i, [C.POINTER(_vp), C.c_char_p]),
    "lpp_gguf_close": (_i, [_vp]),
    "lpp_gguf_config": (_i, [_vp, C.POINTER(LppConfig)]),
    "lpp_gguf_tensor": (_i, [_vp, C.c_char_p, C.POINTER(_vp), _ip, C.POINTER(_sz)]),
    "lpp_model_load_gguf": (_i, [C.POINTER(_vp), _vp]),
    "lpp_tokenizer_load": (_i, [C.POINTER(_vp), C.c_char_p, _i]),
    "lpp_tokenizer_from_gguf": (_i, [C.POINTER(_vp), _vp]),
    "lpp_tokenizer_free": (_i, [_vp]),
    "lpp_tokenizer_info": (_i, [_vp, _ip, _ip, _ip]),
    "lpp_tokenizer_encode": (_i, [_vp, C.c_char_p, _vp, _i, _ip]),
    "lpp_tokenizer_decode": (_i, [_vp, _i, C.c_char_p, _sz]),
    # C. runtime
    "lpp_last_error": (C.c_char_p, []),
    "lpp_version": (C.c_char_p, []),
    "lpp_device_count": (_i, [_ip]),
    "lpp_init": (_i, [_i]),
    "lpp_set_stream": (_i, [_vp]),
    "lpp_get_stream": (_i, [C.POINTER(_vp)]),
    "lpp_synchronize": (_i, []),
    "lpp_malloc": (_i, [C.POINTER(_vp), _sz]),
    "lpp_free": (_i, [_vp]),
    "lpp_memset": (_i, [_vp, _i, _sz]),
    "lpp_memcpy_h2d": (_i, [_vp, _vp, _sz]),
    "lpp_memcpy_d2h": (_i, [_vp, _vp, _sz]),
    "lpp_memcpy_d2d": (_i, [_vp, _vp, _sz]),
    "lpp_malloc_host": (_i, [C.POINTER(_vp), _sz]),
    "lpp_free_host": (_i, [_vp]),
    "lpp_device_info": (_i, [C.c_char_p, _sz, _ip, C.POINTER(_sz)]),
    "lpp_set_test_option": (_i, [_i, _i]),
    "lpp_get_test_option": (_i, [_i, _ip]),
    "lpp_synth_normal_f32": (_i, [_vp, _sz, _u64, _u64, _f]),
    "lpp_synth_normal_f16": (_i, [_vp, _sz, _u64, _u64, _f]),
    "lpp_synth_uniform_f32": (_i, [_vp, _sz, _u64, _u64]),
    "lpp_synth_token_ids": (_i, [_vp, _sz, _u64, _i]),
    "lpp_f16_to_f32_host": (_i, [_vp, _vp, _sz]),
    "lpp_f32_to_f16_host": (_i, [_vp, _vp, _sz]),
}

_lib = None


def load() -> C.CDLL:
    """Load liblpp_hip.so and bind every declared entry point."""
    global _lib
    if _lib is not None:
        return _lib
    if not LIB_PATH.exists():
        raise ImportError(
            f"{LIB_PATH} is missing: build it with `make -C {PKG_DIR / 'csrc'}` "
            "(or __graft_entry__.build()); there is no fallback implementation")
    lib = C.CDLL(os.fspath(LIB_PATH))
    for name, (restype, argtypes) in SIGNATURES.items():
        fn = getattr(lib, name)  # AttributeError if the symbol is not exported
        fn.restype = restype
        fn.argtypes = argtypes
    _lib = lib
    return lib


def check(status: int) -> None:
    if status != LPP_OK:
        raise LppError(status, load().lpp_last_error().decode(errors="replace"))


def device_count() -> int:
    n = C.c_int(0)
    check(load().lpp_device_count(C.byref(n)))
    return n.value


def _host_ptr(a: np.ndarray) -> C.c_void_p:
    return C.c_void_p(a.ctypes.data)


class DeviceBuffer:
    """A raw device allocation (lpp_malloc) with numpy round trips."""

    def __init__(self, nbytes: int):
        self.nbytes = int(nbytes)
        p = C.c_void_p()
        check(load().lpp_malloc(C.byref(p), self.nbytes))
        self.ptr = p.value or 0

    @classmethod
    def from_numpy(cls, a: np.ndarray) -> "DeviceBuffer":
        a = np.ascontiguousarray(a)
        buf = cls(a.nbytes)
        if a.nbytes:
            check(load().lpp_memcpy_h2d(buf.ptr, _host_ptr(a), a.nbytes))
        return buf

    def upload(self, a: np.ndarray, byte_offset: int = 0) -> None:
        a = np.ascontiguousarray(a)
        assert byte_offset + a.nbytes <= self.nbytes
        if a.nbytes:
            check(load().lpp_memcpy_h2d(self.ptr + byte_offset, _host_ptr(a), a.nbytes))

    def to_numpy(self, dtype, count: int | None = None, byte_offset: int = 0) -> np.ndarray:
        dtype = np.dtype(dtype)
        if count is None:
            count = (self.nbytes - byte_offset) // dtype.itemsize
        out = np.empty(count, dtype=dtype)
        if out.nbytes:
            check(load().lpp_memcpy_d2h(_host_ptr(out), self.ptr + byte_offset, out.nbytes))
        return out

    def at(self, byte_offset: int) -> int:
        return self.ptr + byte_offset

    def free(self) -> None:
        if self.ptr:
            load().lpp_free(self.ptr)
            self.ptr = 0

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass


def synchronize() -> None:
    check(load().lpp_synchronize())


def set_test_option(option: int, value: int) -> None:
    check(load().lpp_set_test_option(option, value))


def get_test_option(option: int) -> int:
    v = C.c_int(0)
    check(load().lpp_get_test_option(option, C.byref(v)))
    return v.value


def reset_test_options() -> None:
    for option, value in OPT_DEFAULTS.items():
        set_test_option(option, value)


# ---- synthetic data -------------------------------------------------------------

def synth_normal_f32(n: int, seed: int, std: float, first_index: int = 0) -> np.ndarray:
    out = np.empty(n, dtype=np.float32)
    check(load().lpp_synth_normal_f32(_host_ptr(out), n, seed, first_index, std))
    return out


def synth_normal_f16(n: int, seed: int, std: float, first_index: int = 0) -> np.ndarray:
    """binary16 bit patterns (uint16)."""
    out = np.empty(n, dtype=np.uint16)
    check(load().lpp_synth_normal_f16(_host_ptr(out), n, seed, first_index, std))
    return out


def synth_uniform_f32(n: int, seed: int, first_index: int = 0) -> np.ndarray:
    out = np.empty(n, dtype=np.float32)
    check(load().lpp_synth_uniform_f32(_host_ptr(out), n, seed, first_index))
    return out


def synth_token_ids(n: int, seed: int, vocab: int) -> np.ndarray:
    out = np.empty(n, dtype=np.int32)
    check(load().lpp_synth_token_ids(_host_ptr(out), n, seed, vocab))
    return out


def f16_to_f32(bits: np.ndarray) -> np.ndarray:
    bits = np.ascontiguousarray(bits, dtype=np.uint16)
    out = np.empty(bits.shape, dtype=np.float32)
    check(load().lpp_f16_to_f32_host(_host_ptr(out), _host_ptr(bits), bits.size))
    return out


def f32_to_f16(vals: np.ndarray) -> np.ndarray:
    vals = np.ascontiguousarray(vals, dtype=np.float32)
    out = np.empty(vals.shape, dtype=np.uint16)
    check(load().lpp_f32_to_f16_host(_host_ptr(out), _host_ptr(vals), vals.size))
    return out
