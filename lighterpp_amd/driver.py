"""Command-line driver over liblpp_hip.so: what src/main.cpp does with a llama2.c
checkpoint or a GGUF file (F32 / F16).

    python -m lighterpp_amd.driver model.bin|model.gguf [--tokenizer tokenizer.bin] [--prompt "text"]
                                   [--prompt-ids 1,15,7] [--steps 200] [--temperature 0.8] [--seed 1]
                                   [--path persistent]

With a tokenizer (a llama2.c tokenizer file, or the vocabulary inside a GGUF file) text goes
in and comes out; without one, ids do.

Prefill by decode, 64-entry sliding penalty window (1.1 while reading the prompt,
1.05 while generating), stop at position --steps or at an end-of-sequence id, then the
statistics block of main.cpp:228-232.
"""
from __future__ import annotations

import argparse
import sys

import numpy as np

from . import capi
from .model import Checkpoint, Gguf, Model, Tokenizer

PATHS = {"ops": capi.PATH_OPS, "fused": capi.PATH_FUSED, "persistent": capi.PATH_PERSISTENT}


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(prog="lighterpp_amd.driver", description=__doc__.split("\n\n")[0])
    ap.add_argument("checkpoint", help="llama2.c .bin file or GGUF file")
    ap.add_argument("--tokenizer", default=None, help="llama2.c tokenizer file (default for GGUF: the embedded vocabulary)")
    ap.add_argument("--prompt", default=None, help="prompt text (needs a tokenizer)")
    ap.add_argument("--prompt-ids", default="", help="comma-separated token ids (default: the single id 1)")
    ap.add_argument("--steps", type=int, default=200, help="last position + 1 (main.cpp:155)")
    ap.add_argument("--temperature", type=float, default=0.8)
    ap.add_argument("--seed", type=int, default=1, help="seed of the per-step uniform draws")
    ap.add_argument("--path", default="persistent", choices=list(PATHS))
    ap.add_argument("--batched-prefill", action="store_true",
                    help="fill the cache for the prompt in one pass per 512 ids (lpp_run_batched_prefill) instead of by decode")
    args = ap.parse_args(argv)

    capi.check(capi.load().lpp_init(0))
    with open(args.checkpoint, "rb") as f:
        is_gguf = f.read(4) == b"GGUF"  # is_gguf_file, loader.cpp:200-211
    ck = Gguf(args.checkpoint) if is_gguf else Checkpoint(args.checkpoint)
    c = ck.config
    print("--- Model Configuration ---")
    print(f"Dim: {c.dim}\nHidden Dim: {c.hidden_dim}\nLayers: {c.n_layers}\nHeads: {c.n_heads}\nKV Heads: {c.n_kv_heads}")
    print(f"Vocab: {c.vocab_size}\nSeq Len: {c.seq_len}\nRoPE Base: {c.rope_base:.0f}\nTemperature: {args.temperature:.2f}")
    model = Model.from_gguf(ck) if is_gguf else Model.from_checkpoint(ck)
    try:
        model.set_path(PATHS[args.path])
    except capi.LppError as e:  # e.g. fp32 rows wider than the persistent kernel takes
        if e.status != capi.LPP_ERR_UNSUPPORTED or args.path != "persistent":
            raise
        print(f"note: {e}; using the fused graph path")
        model.set_path(PATHS["fused"])
    tok = None
    if args.tokenizer:
        tok = Tokenizer.load(args.tokenizer, c.vocab_size)
    elif is_gguf:
        try:
            tok = Tokenizer.from_gguf(ck)
        except capi.LppError:
            tok = None  # main.cpp:78-82: ids are printed instead
    prompt = [int(t) for t in args.prompt_ids.split(",") if t.strip()] or None
    if args.prompt is not None:
        if tok is None:
            ap.error("--prompt needs a tokenizer")
        prompt = tok.encode(args.prompt, 2048)  # main.cpp:140-146
        print(f"Encoded {len(prompt)} tokens.")
    steps = min(args.steps, c.seq_len)
    uniforms = capi.synth_uniform_f32(max(steps, len(prompt or [1])), args.seed)  # one draw per position, prompt included
    print("\n--- Running Inference ---")
    tokens, res = model.run(prompt, steps, args.temperature, 1.0, uniforms, batched_prefill=args.batched_prefill)
    if tok is not None:
        shown = list(prompt or [1]) + [int(t) for t in tokens]  # main.cpp:175-176, 191-192, 215-221
        sys.stdout.buffer.write(b"".join(tok.decode(t) for t in shown) + b"\n")
        sys.stdout.flush()
    else:
        print(" ".join(str(int(t)) for t in tokens))
    print("\n--- Statistics ---")
    print(f"Tokens generated: {res.reported_count}")
    print(f"Elapsed time: {res.wall_seconds:.2f} s")
    if res.wall_seconds > 0:
        print(f"Tokens per second: {res.reported_count / res.wall_seconds:.2f} tok/s")
    model.close()
    ck.close()
    return 0


if __name__ == "__main__":
    sys.exit(main())
