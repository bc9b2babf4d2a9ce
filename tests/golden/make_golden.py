"""Writes tests/golden/ref_cpu_path.npz from the COMPILED REFERENCE
(oracle/_ref/liblpp_ref.so = the reference's own ops.cpp + model.cpp, built by
oracle/Makefile).  Run in the build container, where /root/reference exists:

    make -C oracle && python tests/golden/make_golden.py

The fixture holds data only: seeds, shapes, the uniform draws that were fed to
the sampler, and what the reference computed (logit bit patterns, token ids,
cache contents).  tests/test_oracle_golden.py replays the same inputs through
the restated oracle and demands bit equality.

Covers what no test of the reference pins: attention with grouped KV heads,
transformer_block, forward over several positions (exact fp32 summation order),
the KV-cache scatter, and sample() with its per-occurrence penalty, both greedy
and with the plain-CDF draw, plus the nucleus branch.
"""
from __future__ import annotations

import ctypes as C
import sys
from pathlib import Path

import numpy as np

ROOT = Path(__file__).resolve().parent.parent.parent
sys.path.insert(0, str(ROOT))
sys.path.insert(0, str(ROOT / "tests"))

import oracle_binding as ob  # noqa: E402
from lighterpp_amd import Shape, capi, synth_tensor  # noqa: E402

OUT = Path(__file__).resolve().parent / "ref_cpu_path.npz"

CASES = {
    # name: (Shape, seed)
    "gqa4_fp32": (Shape(64, 160, 3, 8, 2, 320, 32, 10000.0, fp16=False, tied=True), 11),
    "mha_fp32": (Shape(48, 96, 2, 4, 4, 200, 24, 10000.0, fp16=False, tied=False), 12),
    "gqa8_f16vals": (Shape(128, 256, 2, 16, 2, 512, 40, 500000.0, fp16=True, tied=True), 13),
}


def weights_f32(shape: Shape, seed: int) -> dict:
    """fp32 host weights as the reference's loaders would hold them: for an fp16
    model the binary16 values widened exactly."""
    out = {}
    for t in range(12):
        a = synth_tensor(shape, t, seed)
        if a.dtype == np.uint16:
            a = capi.f16_to_f32(a)
        out[t] = np.ascontiguousarray(a, dtype=np.float32)
    return out


def bits(a: np.ndarray) -> np.ndarray:
    return np.ascontiguousarray(a, dtype=np.float32).view(np.uint32).copy()


def history_push(hist: list, cap: int, tok: int) -> None:
    if len(hist) < cap:
        hist.append(tok)
    else:
        hist.pop(0)
        hist.append(tok)


def run_case(name: str, shape: Shape, seed: int, store: dict) -> None:
    w = weights_f32(shape, seed)
    checksum = np.uint64(0)
    for t in range(12):
        checksum ^= np.bitwise_xor.reduce(w[t].reshape(-1).view(np.uint32).astype(np.uint64) * np.uint64(t + 1))
    store[f"{name}/weights_xor"] = np.array([checksum], dtype=np.uint64)
    prompt = capi.synth_token_ids(4, seed + 100, shape.vocab_size)
    store[f"{name}/prompt"] = prompt

    # 1. greedy: prompt fed token by token, then generated tokens fed back.
    m = ob.RefModel(shape, w)
    steps = min(20, shape.seq_len)
    toks, logit_bits = [], []
    tok = int(prompt[0])
    for pos in range(steps):
        nxt = m.forward(tok, pos, 0.0, 1.0, 1.0, None)
        logit_bits.append(bits(m.buf("logits")))
        toks.append(nxt)
        tok = int(prompt[pos + 1]) if pos + 1 < len(prompt) else nxt
    store[f"{name}/greedy_tokens"] = np.array(toks, dtype=np.int32)
    store[f"{name}/greedy_logit_bits"] = np.stack(logit_bits)
    store[f"{name}/key_cache_bits"] = bits(m.buf("key_cache"))
    store[f"{name}/value_cache_bits"] = bits(m.buf("value_cache"))
    store[f"{name}/x_bits"] = bits(m.buf("x"))
    m.close()

    # 2. sampled: temperature 0.8, penalty 1.1, 8-entry sliding window, plain CDF.
    #    sample() draws rand()/RAND_MAX itself; replay the same libc stream first to
    #    learn the draws, then reseed and run.
    lib = ob.ref()
    m = ob.RefModel(shape, w)
    lib.ref_srand(4242 + seed)
    draws = np.array([lib.ref_next_uniform() for _ in range(steps)], dtype=np.float32)
    lib.ref_srand(4242 + seed)
    hist, toks = [], []
    tok = int(prompt[0])
    history_push(hist, 8, tok)
    for pos in range(steps):
        nxt = m.forward(tok, pos, 0.8, 1.0, 1.1, hist)
        toks.append(nxt)
        tok = nxt
        history_push(hist, 8, tok)
    store[f"{name}/sampled_draws"] = draws
    store[f"{name}/sampled_tokens"] = np.array(toks, dtype=np.int32)
    store[f"{name}/sampled_final_probs_bits"] = bits(m.buf("logits"))
    m.close()


def sampler_cases(store: dict) -> None:
    """sample() alone on hand-built logits: duplicates in the window, ties,
    negative logits, out-of-range ids, nucleus branch."""
    lib = ob.ref()
    rng = np.random.default_rng(7)
    cases = []
    base = (rng.standard_normal(97) * 3).astype(np.float32)
    base[10] = base[40] = base.max() + 1.0  # tie for the maximum: first index must win
    windows = [
        [],
        [5, 5, 5, 10, 96, 0],
        [10, 40, 10, 40, 10, -3, 1000, 96],
        list(range(20)) + [3, 3, 3, 3],
    ]
    for wi, win in enumerate(windows):
        for (temp, topp, pen) in [(0.0, 1.0, 1.3), (0.7, 1.0, 1.3), (1.0, 0.0, 1.0), (1.5, 1.0, 2.0),
                                  (0.9, 0.8, 1.1), (1.0, 0.3, 1.0)]:
            seed = 1000 + 17 * wi + int(temp * 10) + int(topp * 100)
            lib.ref_srand(seed)
            r = lib.ref_next_uniform()
            lib.ref_srand(seed)
            lg = base.copy()
            h = np.array(win, dtype=np.int32)
            tok = lib.ref_sample(lg, lg.size, temp, topp, pen, h.ctypes.data if h.size else None, int(h.size))
            cases.append((win, temp, topp, pen, r, tok, lg))
    store["sampler/base_logits"] = base
    store["sampler/n"] = np.array([len(cases)], dtype=np.int32)
    for i, (win, temp, topp, pen, r, tok, lg) in enumerate(cases):
        store[f"sampler/{i}/window"] = np.array(win, dtype=np.int32)
        store[f"sampler/{i}/params"] = np.array([temp, topp, pen, r], dtype=np.float32)
        store[f"sampler/{i}/token"] = np.array([tok], dtype=np.int32)
        store[f"sampler/{i}/after_bits"] = bits(lg)


def main() -> None:
    if not ob.have_ref():
        raise SystemExit("oracle/_ref/liblpp_ref.so is missing: run `make -C oracle` where /root/reference exists")
    store: dict = {}
    for name, (shape, seed) in CASES.items():
        run_case(name, shape, seed, store)
    sampler_cases(store)
    np.savez_compressed(OUT, **store)
    print(f"wrote {OUT} ({OUT.stat().st_size} bytes, {len(store)} arrays)")


if __name__ == "__main__":
    main()
