"""Trace replay: feeds given token ids through the model step by step and writes logits.
It samples nothing and has no forward pass, cache or loader of its own: it drives
`load_model`, `Engine.step` and the cache that generation uses.

    trace_run --model DIR --dtype bfloat16|float32 --out DIR --max-tokens N

Standard input, one JSON object a line:
    {"step": 0, "entries": [{"id": "a", "tokens": [5, 17, 3], "want": [0, 2]}], "end": []}
For a step in which something is wanted, `<out>/<step>.f32` holds the logits at the wanted
places, in the order of the entries and of `want`, as little-endian float32 [wanted, vocab].
After every step a line `done <step>` is printed and flushed.

The nearest things in the reference are its recording mock engine
(src/conversation.rs:586-613 of yusiwen/minfer) and its logits dump
(src/models/qwen2/graph.rs:372-399).
"""
from __future__ import annotations

import argparse
import json
import os
import sys

import numpy as np


def parse_args(argv=None):
    ap = argparse.ArgumentParser(prog="trace_run", description=__doc__.split("\n\n")[0])
    ap.add_argument("--model", required=True, help="folder with config.json and model.safetensors")
    ap.add_argument("--dtype", required=True, choices=["bfloat16", "float32"])
    ap.add_argument("--out", required=True, help="folder for <step>.f32 files")
    ap.add_argument("--max-tokens", type=int, required=True,
                    help="most tokens live requests hold at any time (each rounded up to 64)")
    ap.add_argument("--device", default="cuda:0")
    return ap.parse_args(argv)


def run(args, stdin=None, stdout=None) -> int:
    stdin = stdin or sys.stdin
    stdout = stdout or sys.stdout
    import torch
    from .engine import Engine, load_model
    if args.dtype == "float32":
        # nothing here uses a library product, but make sure none could run in a reduced mode
        torch.backends.cuda.matmul.allow_tf32 = False
    os.makedirs(args.out, exist_ok=True)
    model = load_model(args.model, dtype=args.dtype, device=args.device)
    engine = Engine(model, max_tokens=max(64, args.max_tokens))
    slots = {}                                  # request id -> cache slot
    for line in stdin:
        line = line.strip()
        if not line:
            continue
        rec = json.loads(line)
        step, entries = rec["step"], rec.get("entries", [])
        if entries:
            for e in entries:
                if e["id"] not in slots:
                    slots[e["id"]] = engine.new_sequence()
            want = [list(e.get("want", [])) for e in entries]
            logits = engine.step([slots[e["id"]] for e in entries],
                                 [list(e["tokens"]) for e in entries], want)
            if logits.shape[0] > 0:
                arr = logits.detach().to("cpu").numpy().astype("<f4", copy=False)
                path = os.path.join(args.out, f"{step}.f32")
                with open(path + ".tmp", "wb") as f:
                    f.write(np.ascontiguousarray(arr).tobytes())
                os.replace(path + ".tmp", path)
        for rid in rec.get("end", []):
            if rid in slots:
                engine.end_sequence(slots.pop(rid))
        stdout.write(f"done {step}\n")
        stdout.flush()
    return 0


def main(argv=None) -> int:
    return run(parse_args(argv))


if __name__ == "__main__":
    sys.exit(main())
