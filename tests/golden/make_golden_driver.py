"""Writes tests/golden/ref_driver.json from the REFERENCE'S OWN EXECUTABLE
(oracle/_ref/lighterpp_ref = src/main.cpp and the six source files it needs,
compiled by oracle/Makefile).  Run in the build container, where /root/reference
exists:

    make -C oracle && python tests/golden/make_golden_driver.py

For each case a tiny seeded llama2.c checkpoint and a tokenizer file whose
vocabulary is one distinct printable character per id are written to a scratch
directory, the executable is run greedily (temperature 0) with and without a
prompt, and the characters it printed are mapped back to ids.  The fixture holds
data only: shape, weight seed, prompt ids as the reference's tokenizer encoded
them, the ids it printed and its "Tokens generated" figure.
tests/test_driver_cpu.py replays the same checkpoints through the oracle's
restatement of the loop (orc_run) and demands the same ids.

Covers what nothing else pins: prefill-by-decode, which penalty applies where, the
sliding 64-entry window (runs longer than 64 positions), the end-of-sequence
stop, and main.cpp's own count of generated tokens.
"""
from __future__ import annotations

import json
import re
import struct
import subprocess
import sys
import tempfile
from pathlib import Path

import numpy as np

ROOT = Path(__file__).resolve().parent.parent.parent
sys.path.insert(0, str(ROOT))
sys.path.insert(0, str(ROOT / "tests"))

import oracle_binding as ob  # noqa: E402
from lighterpp_amd import Shape, synth_tensor, write_checkpoint  # noqa: E402

OUT = Path(__file__).resolve().parent / "ref_driver.json"

# One character per id; none of them is '<', '>' or a blank, no entry is the
# concatenation of two others, so the reference's encoder maps a prompt to one id
# per character and merges nothing.  (Ids 2 -- end of sequence -- and 1 keep an
# ordinary character: vocab[1] is not "<s>", so no BOS is prepended.)
ALPHABET = "abcdefghijklmnopqrstuvwxyzABCDEFGHIJKLMNOPQRSTUVWXYZ0123456789+-*/=%&#@!?$^~|_.,;:"

CASES = {
    # name: (Shape, weight seed, prompt text or None)
    "bos_only": (Shape(64, 96, 2, 4, 2, 40, 200, 10000.0, fp16=False, tied=True), 21, None),
    "prompt_short": (Shape(64, 96, 2, 4, 2, 40, 200, 10000.0, fp16=False, tied=True), 22, "hello"),
    "prompt_long_window": (Shape(64, 160, 2, 8, 2, 80, 200, 10000.0, fp16=False, tied=True), 23,
                           "thequickbrownfoxjumpsoverthelazydogTHEQUICKBROWNFOXJUMPSOVERTHELAZYDOG0123456789"),
    "mha": (Shape(32, 64, 3, 4, 4, 64, 200, 10000.0, fp16=False, tied=True), 24, "abcABC"),
    # twelve ids only: id 2 (end of sequence) turns up during generation and stops the loop,
    # once early and once after the window has started to slide
    "eos_early": (Shape(32, 64, 2, 4, 2, 12, 200, 10000.0, fp16=False, tied=True), 32, "fghij"),
    "eos_after_window_slides": (Shape(32, 64, 2, 4, 2, 12, 200, 10000.0, fp16=False, tied=True), 37, "fghij"),
}


def write_tokenizer(path: Path, vocab: int) -> None:
    """The layout load_tokenizer reads (tokenizer.cpp:15-55): max length, then per id
    a score, a length and the bytes."""
    with open(path, "wb") as f:
        f.write(struct.pack("<i", 1))
        for i in range(vocab):
            s = ALPHABET[i].encode()
            f.write(struct.pack("<fi", 0.0, len(s)))
            f.write(s)


def main() -> None:
    assert ob.REF_EXE.exists(), "build the reference first: make -C oracle"
    out = {}
    with tempfile.TemporaryDirectory() as tmp:
        tmp = Path(tmp)
        for name, (shape, seed, prompt) in CASES.items():
            assert shape.vocab_size <= len(ALPHABET)
            weights = {t: synth_tensor(shape, t, seed) for t in range(12)}
            ck, tk = tmp / f"{name}.bin", tmp / f"{name}.tok"
            write_checkpoint(ck, shape, weights)
            write_tokenizer(tk, shape.vocab_size)
            cmd = [str(ob.REF_EXE), str(ck), str(tk), "0.0"] + (["-p", prompt] if prompt else [])
            text = subprocess.run(cmd, check=True, capture_output=True, text=True).stdout
            body = text.split("--- Running Inference ---\n", 1)[1]
            if prompt:
                body = body.split(" tokens.\n", 1)[1]
            body, stats = body.split("\n\n--- Statistics ---", 1)
            ids = [ALPHABET.index(ch) for ch in body]
            n_prompt = len(prompt) if prompt else 1
            prompt_ids = [ALPHABET.index(ch) for ch in prompt] if prompt else [1]
            assert all(i < shape.vocab_size for i in prompt_ids)
            # the reference prints the prompt's own tokens first (main.cpp:175-176, 191-192)
            assert ids[:n_prompt] == prompt_ids, (ids[:n_prompt], prompt_ids)
            reported = int(re.search(r"Tokens generated: (-?\d+)", stats).group(1))
            out[name] = {
                "shape": [shape.dim, shape.hidden_dim, shape.n_layers, shape.n_heads, shape.n_kv_heads,
                          shape.vocab_size, shape.seq_len],
                "seed": seed,
                "prompt_ids": prompt_ids if prompt else None,
                "steps": 200,
                "generated": ids[n_prompt:],
                "reported_count": reported,
            }
            print(name, "prompt", n_prompt, "generated", len(ids) - n_prompt, "reported", reported)
    OUT.write_text(json.dumps(out, indent=1) + "\n")
    print("wrote", OUT)


if __name__ == "__main__":
    main()
