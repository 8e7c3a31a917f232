"""Trace replay: feed given token ids through the engine step by step and write logits.

It samples nothing and has no forward pass, cache or loader of its own: every
step goes through `Engine.step`, the function that generation uses. Input is
one JSON object per line on standard input:

    {"step": 0, "entries": [{"id": "a", "tokens": [5, 17, 3], "want": [0, 2]}], "end": []}

For a step that wants something, `<out>/<step>.f32` holds the float32 logits
[wanted, vocab] (little-endian) in the order of the entries and of `want`.
After each step a line `done <step>` is printed and flushed.

The reference has no replay program; its nearest hooks are token ids given as the prompt
(crates/cli/src/token_parser.rs:13-26) and logits at every fed position
(crates/backends/backend_common/src/generic_model.rs:808-826).
"""
import argparse
import json
import os
import sys

import numpy as np

from ..errors import HerbertError, RequestError
from .batch import StepEntry
from .engine import Engine


class Replayer:
    def __init__(self, engine, out_dir):
        self.engine = engine
        self.out_dir = out_dir
        self.slots = {}
        os.makedirs(out_dir, exist_ok=True)

    def run_step(self, record):
        try:
            step = record["step"]
            asked = [(e["id"], [int(t) for t in e["tokens"]], [int(j) for j in e.get("want", [])])
                     for e in record.get("entries", [])]
            ended = list(record.get("end", []))
        except (KeyError, TypeError, ValueError) as e:
            raise RequestError(f"a step is an object with \"step\", \"entries\" (each with \"id\", \"tokens\" "
                               f"and \"want\") and \"end\": {type(e).__name__} {e}") from None
        entries = []
        for rid, tokens, want in asked:
            if rid not in self.slots:
                self.slots[rid] = self.engine.alloc_slot()
            entries.append(StepEntry(self.slots[rid], tokens, want))
        if entries:
            logits = self.engine.step(entries)
            if logits is not None:
                arr = logits.detach().to("cpu").numpy().astype("<f4", copy=False)
                arr.tofile(os.path.join(self.out_dir, f"{step}.f32"))
        for rid in ended:
            if rid not in self.slots:
                raise RequestError(f"request {rid!r} ends but never started")
            self.engine.free_slot(self.slots.pop(rid))
        return step


def main(argv=None):
    ap = argparse.ArgumentParser(prog="trace_run", description=__doc__.split("\n\n")[0])
    ap.add_argument("--model", required=True, help="folder with config.json and model.safetensors")
    ap.add_argument("--dtype", required=True, choices=["bfloat16", "float32"])
    ap.add_argument("--out", required=True, help="folder for <step>.f32 files")
    ap.add_argument("--max-tokens", type=int, required=True,
                    help="most tokens live requests hold at any time (each rounded up to 64)")
    args = ap.parse_args(argv)
    try:
        engine = Engine.from_folder(args.model, dtype=args.dtype, max_tokens=args.max_tokens)
        replayer = Replayer(engine, args.out)
        for number, line in enumerate(sys.stdin, 1):
            line = line.strip()
            if not line:
                continue
            try:
                record = json.loads(line)
            except ValueError as e:
                raise RequestError(f"line {number} of the input is not JSON: {e}") from None
            step = replayer.run_step(record)
            print(f"done {step}", flush=True)
    except HerbertError as e:
        print(f"trace_run: {e}", file=sys.stderr, flush=True)
        return 1
    return 0
