"""Driving bin/trace_run as a user would, and building traces from requests."""
import json
import os
import subprocess
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
TRACE_RUN = os.path.join(ROOT, "bin", "trace_run")


def run_trace(folder, dtype, steps, out_dir, max_tokens, vocab, timeout=300):
    """Feed `steps` (dicts) to trace_run one by one; returns {step: array [wanted, vocab]}."""
    os.makedirs(out_dir, exist_ok=True)
    proc = subprocess.Popen(
        [sys.executable, TRACE_RUN, "--model", folder, "--dtype", dtype, "--out", out_dir,
         "--max-tokens", str(max_tokens)],
        stdin=subprocess.PIPE, stdout=subprocess.PIPE, text=True)
    try:
        for rec in steps:
            proc.stdin.write(json.dumps(rec) + "\n")
            proc.stdin.flush()
            line = proc.stdout.readline()
            assert line.strip() == f"done {rec['step']}", f"trace_run said {line!r}"
        proc.stdin.close()
        rc = proc.wait(timeout=timeout)
    finally:
        if proc.poll() is None:
            proc.kill()
    assert rc == 0, f"trace_run exited with {rc}"
    out = {}
    for rec in steps:
        wanted = sum(len(e.get("want", [])) for e in rec["entries"])
        if wanted:
            arr = np.fromfile(os.path.join(out_dir, f"{rec['step']}.f32"), dtype="<f4")
            out[rec["step"]] = arr.reshape(wanted, vocab)
    return out


def collect(steps, outputs):
    """{(request id, position): logits row} from a trace and its outputs."""
    got = {}
    done = {}
    for rec in steps:
        row = 0
        for e in rec["entries"]:
            base = done.get(e["id"], 0)
            for j in e.get("want", []):
                got[(e["id"], base + j)] = outputs[rec["step"]][row]
                row += 1
            done[e["id"]] = base + len(e["tokens"])
    return got


def trace_whole(requests):
    """Each request alone and whole, every position wanted; one after the other."""
    steps = []
    for i, (rid, toks) in enumerate(requests.items()):
        steps.append({"step": i, "entries": [{"id": rid, "tokens": toks,
                                              "want": list(range(len(toks)))}], "end": [rid]})
    return steps


def trace_tail(requests, tail=32):
    """Each request alone: all but the last `tail` tokens whole, then one token a step."""
    steps = []
    n = 0
    for rid, toks in requests.items():
        head = max(1, len(toks) - tail)
        steps.append({"step": n, "entries": [{"id": rid, "tokens": toks[:head],
                                              "want": list(range(head))}], "end": []})
        n += 1
        for p in range(head, len(toks)):
            steps.append({"step": n, "entries": [{"id": rid, "tokens": [toks[p]], "want": [0]}],
                          "end": [rid] if p == len(toks) - 1 else []})
            n += 1
        if head == len(toks):
            steps[-1]["end"] = [rid]
    return steps


def trace_batches(requests, batch_size, prompt_frac=0.5):
    """Batches of unequal lengths, one after another: the prompts (a part of each request)
    in one step, then one token each; shorter requests end earlier, their slots are used
    again by the next batch."""
    steps = []
    n = 0
    items = list(requests.items())
    for b0 in range(0, len(items), batch_size):
        group = items[b0:b0 + batch_size]
        heads = {rid: max(1, int(len(t) * prompt_frac)) for rid, t in group}
        live = {rid: heads[rid] for rid, _ in group}
        toks = dict(group)
        first = {"step": n, "entries": [], "end": []}
        for rid, t in group:
            first["entries"].append({"id": rid, "tokens": t[:heads[rid]],
                                     "want": list(range(heads[rid]))})
            if heads[rid] == len(t):
                first["end"].append(rid)
                del live[rid]
        steps.append(first)
        n += 1
        while live:
            rec = {"step": n, "entries": [], "end": []}
            for rid in list(live):
                p = live[rid]
                rec["entries"].append({"id": rid, "tokens": [toks[rid][p]], "want": [0]})
                live[rid] = p + 1
                if p + 1 == len(toks[rid]):
                    rec["end"].append(rid)
                    del live[rid]
            steps.append(rec)
            n += 1
    return steps


def needed_tokens(steps):
    """The --max-tokens a trace needs: the most tokens held at once, each rounded up to 64."""
    held = {}
    most = 0
    for rec in steps:
        for e in rec["entries"]:
            held[e["id"]] = held.get(e["id"], 0) + len(e["tokens"])
        most = max(most, sum((v + 63) // 64 * 64 for v in held.values()))
        for rid in rec["end"]:
            held.pop(rid, None)
    return most
