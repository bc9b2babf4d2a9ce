"""Where one token's time goes on the persistent decode kernel (LPP_PATH_PERSISTENT).

    python -m lighterpp_amd.timeline [--config c3_llama32_1b_fp16] [--pos 200] [--json]

Runs lpp_trace_token_all (every workgroup writes eight time marks per phase) on
synthetic weights of the named shape and prints, per kind of phase and averaged
over the layers after the first:

  span       from the moment the LAST workgroup has published the phase's inputs to the
             moment the last workgroup has published its outputs (the spans add up to
             the token);
  hand-over  from that first moment to the median workgroup's "inputs received" mark;
  stream     median workgroup: inputs staged -> all its rows multiplied;
  epilogue   median workgroup: rows multiplied -> outputs published;
  skew       last workgroup's publish minus the median workgroup's;
  floor      the phase's weight bytes at 7 TB/s, the rate a plain streaming read reaches.

The closing lines restate the token as  bytes / 7 TB/s  +  hand-overs x mean cost.
Marks cost about half a microsecond each, so a traced token is slower than an
untraced one; the proportions are what the table is for.
"""
from __future__ import annotations

import argparse
import ctypes as C
import json
import sys

import numpy as np

from . import capi
from .model import CONFIGS, Model, Shape

KINDS = ["qkv", "attention", "o-proj", "gate/up", "down"]
STREAM_CEILING = 7.0e12  # bytes/s of a plain non-temporal streaming read on this part


def trace(model: Model, pos: int) -> np.ndarray:
    """[workgroup, phase, mark] in microseconds on workgroup 0's clock; NaN where a mark was not taken."""
    lib = model.lib
    n, marks, nwg = C.c_int(), C.c_int(), C.c_int()
    cap = 1024 * 8 * (5 * model.shape.n_layers + 2)
    arr = (C.c_ulonglong * cap)()
    capi.check(lib.lpp_trace_token_all(model.handle, pos, arr, cap, C.byref(n), C.byref(marks), C.byref(nwg)))
    t = np.ctypeslib.as_array(arr)[: n.value * nwg.value].astype(np.float64).reshape(nwg.value, -1, marks.value) * 0.01
    t[t == 0] = np.nan
    return t


def phase_bytes(shape: Shape, pos: int) -> list:
    w = 2 if shape.fp16 else 4
    d, kv, h = shape.dim, shape.kv_dim, shape.hidden_dim
    return [w * (d + 2 * kv) * d, 2 * 2 * kv * (pos + 1), w * d * d, w * 2 * h * d, w * d * h]


def summarise(shape: Shape, t: np.ndarray, pos: int) -> dict:
    L = shape.n_layers
    pub = t[:, :, 4]
    last_pub = np.nanmax(pub, axis=0)      # per phase
    med_pub = np.nanmedian(pub, axis=0)
    rows = []
    bytes_of = phase_bytes(shape, pos)
    for kind in range(5):
        acc = {k: [] for k in ("span", "handover", "stream", "epilogue", "skew")}
        for layer in range(1, L):
            i = 5 * layer + kind
            start = last_pub[i - 1]
            acc["span"].append(last_pub[i] - start)
            acc["handover"].append(np.nanmedian(t[:, i, 1]) - start)
            if kind != 1:
                acc["stream"].append(np.nanmedian(t[:, i, 3] - t[:, i, 2]))
                acc["epilogue"].append(np.nanmedian(t[:, i, 4] - t[:, i, 3]))
            acc["skew"].append(last_pub[i] - med_pub[i])
        row = {k: (float(np.mean(v)) if v else None) for k, v in acc.items()}
        row["kind"] = KINDS[kind]
        row["floor"] = bytes_of[kind] / STREAM_CEILING * 1e6
        rows.append(row)
    # attention work items (the workgroups that hold one): mark 0 entered, 5 q/k/v received, 2 shared through LDS,
    # 7 context walked, 3 merged, 4 published
    att = {k: [] for k in ("wait_inputs", "share", "walk", "merge", "publish")}
    # GEMV phases, streaming wavefront 0 of every workgroup: mark 5 staged flag seen, 6 last row finished
    gemv = {KINDS[k]: {"flag_after_staged": [], "last_row_after_flag": []} for k in (0, 2, 3, 4)}
    for layer in range(1, L):
        i = 5 * layer + 1
        busy = ~np.isnan(t[:, i, 7])
        if busy.any():
            a = t[busy, i, :]
            att["wait_inputs"].append(np.nanmedian(a[:, 5] - a[:, 0]))
            att["share"].append(np.nanmedian(a[:, 2] - a[:, 5]))
            att["walk"].append(np.nanmedian(a[:, 7] - a[:, 2]))
            att["merge"].append(np.nanmedian(a[:, 3] - a[:, 7]))
            att["publish"].append(np.nanmedian(a[:, 4] - a[:, 3]))
        for k in (0, 2, 3, 4):
            g = t[:, 5 * layer + k, :]
            gemv[KINDS[k]]["flag_after_staged"].append(np.nanmedian(g[:, 5] - g[:, 2]))
            gemv[KINDS[k]]["last_row_after_flag"].append(np.nanmedian(g[:, 6] - g[:, 5]))
    cls, smp = 5 * L, 5 * L + 1
    w = 2 if shape.fp16 else 4
    out = {
        "pos": pos,
        "workgroups": int(t.shape[0]),
        "phases": rows,
        "layer_us": float(sum(r["span"] for r in rows)),
        "layer_floor_us": float(sum(r["floor"] for r in rows)),
        "first_layer_us": float(last_pub[4]),
        "classifier_us": float(last_pub[cls] - last_pub[cls - 1]),
        "classifier_floor_us": w * shape.vocab_size * shape.dim / STREAM_CEILING * 1e6,
        "sampler_us": float(last_pub[smp] - last_pub[cls]),
        "token_us": float(last_pub[smp]),
        "attention_item": {k: (float(np.mean(v)) if v else None) for k, v in att.items()},
        "attention_workgroups": int(np.sum(~np.isnan(t[:, 6, 7]))) if L > 1 else 0,
        "streaming_wavefront": {k: {kk: float(np.mean(vv)) for kk, vv in v.items()} for k, v in gemv.items()},
    }
    n_hand = 5 * L + 1
    total_floor = out["layer_floor_us"] * L + out["classifier_floor_us"]
    out["handovers"] = n_hand
    out["stream_floor_us"] = float(total_floor)
    out["mean_handover_cost_us"] = float((out["token_us"] - total_floor - out["sampler_us"]) / n_hand)
    return out


def render(name: str, s: dict) -> str:
    lines = [f"{name}, position {s['pos']}, {s['workgroups']} workgroups traced; microseconds, mean over layers 1..",
             f"{'phase':10s} {'span':>7s} {'hand-over':>10s} {'stream':>7s} {'epilogue':>9s} {'skew':>6s} {'floor':>7s}"]
    fmt = lambda v: "    -  " if v is None else f"{v:7.2f}"
    for r in s["phases"]:
        lines.append(f"{r['kind']:10s} {fmt(r['span'])} {fmt(r['handover']):>10s} {fmt(r['stream'])} {fmt(r['epilogue']):>9s} "
                     f"{r['skew']:6.2f} {r['floor']:7.2f}")
    a = s["attention_item"]
    if a["walk"] is not None:
        lines.append(f"attention item ({s['attention_workgroups']} workgroups hold one): inputs {a['wait_inputs']:.2f}, shared in LDS "
                     f"{a['share']:.2f}, context walked {a['walk']:.2f}, merged {a['merge']:.2f}, published {a['publish']:.2f}")
    lines.append("streaming wavefront 0 (after the exchange wavefronts' staged mark: flag seen, then last row done): " +
                 "; ".join(f"{k} {v['flag_after_staged']:.2f} + {v['last_row_after_flag']:.2f}" for k, v in s["streaming_wavefront"].items()))
    lines.append(f"layer      {s['layer_us']:7.2f}   (weights of one layer at 7 TB/s: {s['layer_floor_us']:.2f})")
    lines.append(f"first layer {s['first_layer_us']:.2f}; classifier {s['classifier_us']:.2f} (floor {s['classifier_floor_us']:.2f}); "
                 f"sampler {s['sampler_us']:.2f}; token {s['token_us']:.2f}")
    lines.append(f"token = {s['stream_floor_us']:.1f} (bytes / 7 TB/s) + {s['sampler_us']:.1f} (sampler) + "
                 f"{s['handovers']} hand-overs x {s['mean_handover_cost_us']:.2f}")
    return "\n".join(lines)


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--config", default="c3_llama32_1b_fp16", choices=list(CONFIGS))
    ap.add_argument("--pos", type=int, default=200)
    ap.add_argument("--json", action="store_true")
    args = ap.parse_args()
    capi.check(capi.load().lpp_init(0))
    shape = CONFIGS[args.config]
    m = Model(shape)
    m.load_synthetic(1)
    s = summarise(shape, trace(m, args.pos), args.pos)
    print(json.dumps(s) if args.json else render(args.config, s))
    m.close()
    return 0


if __name__ == "__main__":
    sys.exit(main())
