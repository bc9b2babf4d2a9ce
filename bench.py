#!/usr/bin/env python3
"""Batch-1 decode benchmark of liblpp_hip.so on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--config NAME] [--path fused|ops|persistent]

A step is one decoded token: forward() over every layer, classifier and the
fused sampler, on synthetic seeded weights of the named shape, with weights and
KV cache resident in HBM before the clock starts.  The timed region is the
generation loop of the reference's main.cpp (one forward per token, the 4-byte
token copy per token included).  Prints ONE JSON line.

Besides the throughput the line carries
  roofline     the dominant kernel's achieved HBM rate (algorithmic bytes per
               launch / mean launch duration from HIP events on the launch
               stream) against MI355X's 8 TB/s,
  cpu_baseline the reference CPU path (oracle/_ref, the reference's own
               ops.cpp + model.cpp compiled for the host; falls back to the
               restated oracle) timed on a bounded sample of the same workload
               on the host cores of this machine,
  timeline     per-phase microseconds of one traced token of the persistent
               kernel (span, hand-over, streaming, skew, streaming floor) and the
               restatement  token = bytes / 7 TB/s + sampler + hand-overs x mean cost,
  parity       logits of the first decoded positions against the CPU oracle.
"""
from __future__ import annotations

import argparse
import ctypes
import json
import os
import sys
import time
from pathlib import Path

import numpy as np

ROOT = Path(__file__).resolve().parent
sys.path.insert(0, str(ROOT))
sys.path.insert(0, str(ROOT / "tests"))

HBM_PEAK_GBS = 8000.0
# (config, kernel) -> (HBM bytes fetched + written per launch from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE, SHA-256 of
# the kernel's source file when the two counter runs were made).  Hardware counters cannot be read in-process, so
# the figure is a constant; it is quoted only while the kernel's source is the one that was measured, and is null
# (with a note) from the moment the file changes until the two runs are repeated
# (profiles/persistent_decode_<workload>_pmc_hbm_traffic.txt give the commands, one file per configuration).
KERNEL_SOURCES = {"k_decode_dataflow": ROOT / "lighterpp_amd" / "csrc" / "dataflow_decode.hip"}
_MEASURED_SOURCE = "139941b0656e525d92eaab49db8b02a6e9f394abcff588ca3524e4c9bfb94717"
MEASURED_HBM_BYTES_PER_LAUNCH = {
    ("c2_tinyllama_1b_fp16", "k_decode_dataflow"): (2.1260e9, _MEASURED_SOURCE),
    ("c3_llama32_1b_fp16", "k_decode_dataflow"): (2.5143e9, _MEASURED_SOURCE),
    ("c4_llama32_1b_longctx_fp16", "k_decode_dataflow"): (2.8007e9, _MEASURED_SOURCE),
    ("c5_llama3_8b_fp16", "k_decode_dataflow"): (1.5185e10, _MEASURED_SOURCE),
}


def measured_traffic(config: str, kernel: str):
    """(bytes per launch or None, note or None) for the dominant kernel."""
    import hashlib
    entry = MEASURED_HBM_BYTES_PER_LAUNCH.get((config, kernel))
    if entry is None:
        return None, "no counter run for this configuration"
    src = KERNEL_SOURCES.get(kernel)
    if src is None or not src.exists():
        return None, "kernel source not found: counter figure not quoted"
    if hashlib.sha256(src.read_bytes()).hexdigest() != entry[1]:
        return None, "kernel source changed since the counter runs: repeat them"
    return entry[0], None

METRIC = "decode tok/s at batch 1 + % of 8 TB/s HBM roofline, Llama-3.2-1B-shape fp16"

# Workload of each configuration: (prompt tokens, default decode steps, start position, sampler settings)
WORKLOADS = {
    "c1_llama2c_15m_fp32": dict(prompt=8, steps=248, start=0, temperature=0.0, penalty=1.0, history_cap=0),
    "c2_tinyllama_1b_fp16": dict(prompt=16, steps=512, start=0, temperature=0.0, penalty=1.0, history_cap=0),
    "c3_llama32_1b_fp16": dict(prompt=1, steps=512, start=0, temperature=0.8, penalty=1.1, history_cap=64),
    "c4_llama32_1b_longctx_fp16": dict(prompt=1, steps=256, start=8192, temperature=0.0, penalty=1.0,
                                       history_cap=0),
    "c5_llama3_8b_fp16": dict(prompt=32, steps=1024, start=0, temperature=0.0, penalty=1.0, history_cap=0),
}
SEED = 20251


def log(msg: str) -> None:
    print(f"[bench] {msg}", file=sys.stderr, flush=True)


def prefill_cache(model, shape, upto: int) -> None:
    """Config 4: K/V of positions [0, upto) filled with binary16 N(0, 1)."""
    from lighterpp_amd import capi
    hs, nkv, L, seq = shape.head_size, shape.n_kv_heads, shape.n_layers, shape.seq_len
    for which, buf in ((0, capi.B_KEY_CACHE), (1, capi.B_VALUE_CACHE)):
        for layer in range(L):
            for h in range(nkv):
                a = capi.synth_normal_f16(upto * hs, SEED * 7 + which, 1.0, first_index=(layer * nkv + h) * seq * hs)
                model.write_buffer(buf, a, byte_offset=((layer * nkv + h) * seq * hs) * 2)


def cpu_baseline(shape, weights, wl, first_token, start, budget_s: float, cache=None):
    """Times the CPU path on a bounded sample of the workload.  Prefers the compiled
    reference; otherwise the restated oracle.  cache: (K, V) binary16 bit patterns of a workload that starts on a
    pre-filled cache (config 4); the CPU path gets the same values, widened exactly."""
    import oracle_binding as ob
    from lighterpp_amd import capi
    cores = os.cpu_count() or 1
    kind = "reference" if ob.have_ref() else "port"
    t_build = time.time()
    if kind == "reference":
        w32 = {t: (capi.f16_to_f32(a) if a.dtype == np.uint16 else np.ascontiguousarray(a, np.float32))
               for t, a in weights.items()}
        cpu = ob.RefModel(shape, w32)
        step = lambda tok, pos, hist: cpu.forward(tok, pos, wl["temperature"], 1.0, wl["penalty"], hist)
    else:
        cpu = ob.OracleModel(shape, weights, fp16=shape.fp16)
        step = lambda tok, pos, hist: cpu.forward(tok, pos, wl["temperature"], 1.0, wl["penalty"], hist, 0.5)
    if start > 0 and cache is not None:
        cpu.buf("key_cache")[:] = capi.f16_to_f32(cache[0])
        cpu.buf("value_cache")[:] = capi.f16_to_f32(cache[1])
    log(f"cpu baseline ({kind}) ready in {time.time() - t_build:.1f}s")
    tok, hist, n = first_token, [first_token], 0
    t0 = time.perf_counter()
    while True:
        tok = step(tok, start + n, hist if wl["history_cap"] else None)
        if wl["history_cap"]:
            hist = (hist + [tok])[-wl["history_cap"]:]
        n += 1
        el = time.perf_counter() - t0
        if el >= budget_s or n >= 256 or start + n >= shape.seq_len:
            break
    cpu.close()
    return dict(value=round(n / el, 4), unit="tok/s", cores=1, host_cores=cores, kind=kind,
                sample=f"{n} decode steps from position {start} of the same workload, single thread, {el:.1f}s")


def parity_check(model, shape, weights, prompt, n_steps: int, start: int):
    """Teacher-forced logits comparison against the oracle from the workload's own first position:
    the prompt ids, then the oracle's greedy ids.  A workload that starts on a pre-filled cache
    (config 4) gets the same cache contents on both sides, widened exactly for the oracle."""
    import oracle_binding as ob
    from lighterpp_amd import capi
    o = ob.OracleModel(shape, weights, fp16=shape.fp16, kv_round_f16=True)
    model.reset()
    if start > 0:
        prefill_cache(model, shape, start)
        o.buf("key_cache")[:] = capi.f16_to_f32(model.buffer(capi.B_KEY_CACHE))
        o.buf("value_cache")[:] = capi.f16_to_f32(model.buffer(capi.B_VALUE_CACHE))
    tok, worst, agree = int(prompt[0]), 0.0, 0
    for i in range(n_steps):
        pos = start + i
        nxt = model.forward(tok, pos, 0.0)
        want = o.forward_logits(tok, pos)
        got = model.buffer(capi.B_LOGITS)
        worst = max(worst, float(np.max(np.abs(got - want)) / np.max(np.abs(want))))
        agree += int(nxt == int(np.argmax(want)))
        tok = int(prompt[i + 1]) if i + 1 < len(prompt) else int(np.argmax(want))
    o.close()
    return dict(steps=n_steps, first_pos=start, max_rel_logit_err=worst, greedy_agreement=agree / n_steps, tolerance=2e-3,
                checker="oracle (CPU restatement, binary16 KV store)")


MFMA_F16_PEAK_TFLOPS = 2500.0


def bench_prefill(args, model, shape, name, cus) -> int:
    """Batched prefill of N ids from position 0 (lpp_prefill): K repetitions after W warm-up ones.
    A step is one prefill of the whole prompt; the line's value is prompt ids per second."""
    from lighterpp_amd import capi
    n = min(args.prefill, shape.seq_len)
    if not model.prefill_supported():
        print("bench.py: the batched prefill does not take this model", file=sys.stderr)
        return 2
    ids = capi.synth_token_ids(n, SEED + 1, shape.vocab_size)
    fast = args.prefill_mode == "fast"
    model.set_prefill_mode(capi.PREFILL_FAST if fast else capi.PREFILL_EXACT)
    reps = args.steps if args.steps is not None else 30
    for _ in range(max(args.warmup if args.warmup != 16 else 3, 1)):
        model.prefill(ids, 0)
    capi.synchronize()
    t0 = time.perf_counter()
    for _ in range(reps):
        model.prefill(ids, 0)
    capi.synchronize()
    sec = (time.perf_counter() - t0) / reps
    L, dim, kv, hidden = shape.n_layers, shape.dim, shape.kv_dim, shape.hidden_dim
    # What a prefill owes is the cache: every layer's Wk and Wv products, and Wq, attention, Wo and
    # the feed-forward block of all layers but the last, whose output nothing reads.
    gemm_flops = 2.0 * (L * 2 * kv * dim + (L - 1) * (2 * dim * dim + 3 * hidden * dim)) * n
    att_flops = 4.0 * (L - 1) * shape.n_heads * shape.head_size * n * (n + 1) / 2
    tflops = (gemm_flops + att_flops) / sec / 1e12
    out = dict(metric="batched prefill, prompt ids/s, " + args.config, value=round(n / sec, 1), unit="tok/s", n_gpus=1,
               steps=reps, warmup=max(args.warmup if args.warmup != 16 else 3, 1), ms_per_step=round(sec * 1e3, 3), higher_is_better=True, scaling="weak",
               vs_baseline=None,
               dtype="f32 accumulate over f16 weights, activations rounded to f16 at each GEMM input" if fast
               else "f32 accumulate over f16 weights, activations split hi+lo", data="synthetic",
               config=dict(workload=args.config, prompt_ids=n, chunk=512, prefill_mode=args.prefill_mode),
               roofline=dict(bound="mfma", achieved=round(tflops, 1), peak=MFMA_F16_PEAK_TFLOPS, unit="TFLOP/s",
                             frac=round(tflops / MFMA_F16_PEAK_TFLOPS, 4), traffic=None,
                             note="algorithmic flops of what the cache depends on (the last layer stops at its K/V "
                                  "rows); each product counted once" + ("" if fast else ": the kernel issues two MFMAs "
                                  "per product, for the activation's head and remainder")),
               cpu_baseline=None,
               device=dict(name=name.value.decode(), compute_units=cus.value))
    print(json.dumps(out))
    return 0


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=None)
    ap.add_argument("--warmup", type=int, default=16)
    ap.add_argument("--config", default="c3_llama32_1b_fp16", choices=list(WORKLOADS))
    ap.add_argument("--path", default="persistent", choices=["ops", "fused", "persistent"])
    ap.add_argument("--cpu-seconds", type=float, default=15.0, help="time bound of the CPU baseline sample (0 = skip)")
    ap.add_argument("--parity-steps", type=int, default=3)
    ap.add_argument("--profile-reps", type=int, default=20)
    ap.add_argument("--no-timeline", action="store_true", help="skip the traced token behind the `timeline` object")
    ap.add_argument("--prefill-mode", default="exact", choices=["exact", "fast"],
                    help="with --prefill: activations as binary16 head + remainder (exact) or the head alone (fast)")
    ap.add_argument("--prefill", type=int, default=0, metavar="N",
                    help="time the batched prefill of N prompt ids instead of the decode loop (a second, separate line)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build measures one GPU only (batch-1 decode has no multi-GPU path here); "
              "run with --gpus 1", file=sys.stderr)
        return 2

    from lighterpp_amd import CONFIGS, Model, capi
    lib = capi.load()
    if capi.device_count() < 1:
        print("bench.py: no HIP device visible", file=sys.stderr)
        return 3
    capi.check(lib.lpp_init(0))
    name = ctypes.create_string_buffer(128)
    cus, hbm = ctypes.c_int(), ctypes.c_size_t()
    capi.check(lib.lpp_device_info(name, 128, ctypes.byref(cus), ctypes.byref(hbm)))

    shape = CONFIGS[args.config]
    wl = dict(WORKLOADS[args.config])
    steps = args.steps if args.steps is not None else wl["steps"]
    start = wl["start"] + wl["prompt"] - 1
    steps = min(steps, shape.seq_len - start)
    path = {"ops": capi.PATH_OPS, "fused": capi.PATH_FUSED, "persistent": capi.PATH_PERSISTENT}[args.path]

    t0 = time.time()
    model = Model(shape)
    need_host = args.cpu_seconds > 0 or args.parity_steps > 0
    weights = model.load_synthetic(SEED, keep=need_host)
    log(f"{args.config}: weights resident in HBM after {time.time() - t0:.1f}s "
        f"({shape.matrix_params() / 1e6:.1f} M matrix params)")
    model.set_path(path)
    if args.prefill > 0:
        return bench_prefill(args, model, shape, name, cus)
    prompt = capi.synth_token_ids(max(wl["prompt"], 1), SEED + 1, shape.vocab_size)
    uniforms = capi.synth_uniform_f32(max(steps, args.warmup, 1), SEED + 2)
    temperature, penalty, cap = wl["temperature"], wl["penalty"], wl["history_cap"]

    def run(n_steps: int):
        """Prompt by single forwards (untimed, main.cpp:163-179), then the timed loop."""
        model.reset()
        if wl["start"] > 0:
            prefill_cache(model, shape, wl["start"])
        hist = []
        for i in range(wl["prompt"] - 1):
            hist = (hist + [int(prompt[i])])[-cap:] if cap else []
            model.forward(int(prompt[i]), wl["start"] + i, temperature, 1.0, penalty, hist or None, 0.5)
        first = int(prompt[wl["prompt"] - 1])
        hist = (hist + [first])[-cap:] if cap else []
        return model.generate(first, start, n_steps, temperature=temperature, penalty=penalty, history=hist,
                              history_cap=cap, uniforms=uniforms if temperature != 0.0 else None)

    if args.warmup > 0:
        run(min(args.warmup, steps))
    capi.synchronize()
    t_wall = time.perf_counter()
    tokens, _, stats = run(steps)
    capi.synchronize()
    wall_outer = time.perf_counter() - t_wall  # includes reset/prompt; the figure reported is the loop itself
    sec = stats.wall_seconds
    tok_s = steps / sec
    avg_bytes = float(np.mean([shape.bytes_per_token(p) for p in range(start, start + steps)]))
    log(f"{steps} tokens in {sec * 1e3:.1f} ms -> {tok_s:.1f} tok/s, {avg_bytes * tok_s / 1e9:.0f} GB/s algorithmic "
        f"(outer {wall_outer:.2f}s)")

    # dominant kernel, timed live with HIP events on the launch stream
    roofline = None
    kernels = []
    if True:
        mid = start + steps // 2
        # (operator path: every operator of lpp.h section A timed as a stand-alone launch, as the reference's
        # forward() launches them; the dominant one is the class with the largest share of the token)
        prof = model.profile_kernels(min(mid, shape.seq_len - 1), args.profile_reps if path != capi.PATH_OPS else max(args.profile_reps // 4, 3))
        per_token_ms = sum(n * ms for (_, n, ms, _) in prof)
        kernels = [dict(kernel=k, launches_per_token=n, avg_us=round(ms * 1e3, 3),
                        algorithmic_mb=round(b / 1e6, 3), gbs=round(b / (ms * 1e-3) / 1e9, 1) if ms > 0 else None)
                   for (k, n, ms, b) in prof]
        dom = max(prof, key=lambda p: p[1] * p[2])
        achieved = dom[3] / (dom[2] * 1e-3) / 1e9
        # HBM bytes per launch from hardware counters cannot be read in-process: they come from two
        # rocprofv3 --pmc runs of this script (FETCH_SIZE, WRITE_SIZE, each scaled by what the counter
        # reads for a kernel of known size); the figure is quoted only for the kernel it was measured on.
        traffic, traffic_note = measured_traffic(args.config, dom[0])
        roofline = dict(bound="hbm", kernel=dom[0], achieved=round(achieved, 1), peak=HBM_PEAK_GBS, unit="GB/s",
                        frac=round(achieved / HBM_PEAK_GBS, 4), traffic=traffic,
                        bytes_per_launch=dom[3], avg_launch_us=round(dom[2] * 1e3, 3),
                        sum_of_kernel_times_ms_per_token=round(per_token_ms, 4))
        if traffic_note:
            roofline["traffic_note"] = traffic_note

    # where the token's time goes: per-phase microseconds of one traced token at the window's middle position
    timeline = None
    if path == capi.PATH_PERSISTENT and not args.no_timeline:
        from lighterpp_amd import timeline as tl
        mid = min(start + steps // 2, shape.seq_len - 1)
        summary = tl.summarise(shape, tl.trace(model, mid), mid)
        timeline = dict(position=mid, traced_token_us=round(summary["token_us"], 1),
                        layer_us=round(summary["layer_us"], 2), layer_floor_us=round(summary["layer_floor_us"], 2),
                        phases={r["kind"]: dict(span_us=round(r["span"], 2),
                                                handover_us=round(r["handover"], 2),
                                                stream_us=None if r["stream"] is None else round(r["stream"], 2),
                                                skew_us=round(r["skew"], 2), floor_us=round(r["floor"], 2))
                                for r in summary["phases"]},
                        classifier_us=round(summary["classifier_us"], 1), sampler_us=round(summary["sampler_us"], 1),
                        stream_floor_us=round(summary["stream_floor_us"], 1), handovers=summary["handovers"],
                        mean_handover_cost_us=round(summary["mean_handover_cost_us"], 2),
                        note="every workgroup writes eight time marks per phase: the traced token is slower than "
                             "an untraced one (avg_launch_us), the proportions are what this is for")

    parity = None
    if args.parity_steps > 0:
        parity = parity_check(model, shape, weights, prompt, min(args.parity_steps, shape.seq_len - wl["start"]), wl["start"])
        log(f"parity: {parity}")
    cpu = None
    if args.cpu_seconds > 0:
        cache = None
        if wl["start"] > 0:  # the CPU path starts on the same pre-filled cache
            model.reset()
            prefill_cache(model, shape, wl["start"])
            cache = (model.buffer(capi.B_KEY_CACHE), model.buffer(capi.B_VALUE_CACHE))
        model.close()
        cpu = cpu_baseline(shape, weights, wl, int(prompt[wl['prompt'] - 1]), wl["start"], args.cpu_seconds, cache)
        log(f"cpu baseline: {cpu}")

    out = {
        "metric": METRIC,
        "value": round(tok_s, 2),
        "unit": "tok/s",
        "n_gpus": 1,
        "steps": steps,
        "warmup": args.warmup,
        "ms_per_step": round(sec / steps * 1e3, 5),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32 accumulate over f16 weights" if shape.fp16 else "f32",
        "data": "synthetic",
        "config": {"workload": args.config, "path": args.path, "dim": shape.dim, "hidden_dim": shape.hidden_dim,
                   "n_layers": shape.n_layers, "n_heads": shape.n_heads, "n_kv_heads": shape.n_kv_heads,
                   "vocab_size": shape.vocab_size, "start_pos": start, "temperature": temperature,
                   "penalty": penalty, "history_window": cap, "weights": "N(0,0.02) seeded, norm gains 1"},
        "hbm": {"algorithmic_bytes_per_token": round(avg_bytes), "achieved_gbs": round(avg_bytes * tok_s / 1e9, 1),
                "peak_gbs": HBM_PEAK_GBS, "frac_of_peak": round(avg_bytes * tok_s / 1e9 / HBM_PEAK_GBS, 4),
                "device_ms_per_token": round(stats.device_ms / steps, 5)},
        "roofline": roofline,
        "timeline": timeline,
        "cpu_baseline": cpu,
        "parity": parity,
        "kernels": kernels,
        "device": {"name": name.value.decode(), "compute_units": cus.value},
        "first_tokens": tokens[:8].tolist(),
    }
    print(json.dumps(out), flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
