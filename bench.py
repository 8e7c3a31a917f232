"""Decode and prefill throughput of the Qwen3-8B shape (BASELINE.json configs[2]) on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--layers L] [--batch B] [--context C]

One JSON line: `value` is decoded tokens a second at batch 8 with every sequence holding
`context` tokens; `prefill` is one 2,048-token prompt; `roofline` prices the decode step
against HBM. `points` (flat, numbers only) holds, for batch 1, 8 and 64: tokens a second,
ms a step, GB/s and the fraction of 8 TB/s at the full context (`decode_b1`, `decode_b1_ms`,
`decode_b1_gbs`, `decode_b1_frac`), the same at a context of 512 (`..._ctx512...`) and the mean
over a decode from 512 to the full context (`..._mean...`, from steps timed at a few contexts
in between); and the other two workloads of the benchmark description through the generation
loop (`qwen3_1p7b_...`, `qwen3_32b_...`); `decode_b8_host_between_steps` is the headline's step
with the host reading each step's tokens before it starts the next; `decode_b16_unequal_lengths` is a batch of one
sequence at the full context beside fifteen of a sixteenth of it; and, unless --no-long, further sizes and
lengths: decode at batch 8 at 16,384 and 32,768 tokens of context, at batch 64 at 16,384 (155 GB of keys and
values: 32,768 would not fit beside the weights), at batch 128 and 256 at the full context, and prompts of 8,192,
16,384 and 32,768 tokens fed in chunks of 8,192 (`decode_b8_ctx16384...`, `decode_b128...`, `prefill_8192`,
`prefill_8192_frac`, ...). Weights are random, token ids are random, and the
cache below the timed steps is filled by real prefill steps of random prompts. A timed decode
step is what the generation loop does for a token: the step function (a HIP-graph replay), the
greedy choice on the GPU, and the chosen tokens read by the host, which as in that loop reads
the tokens of a step while the next step, fed from the GPU, already runs.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_GBS = 8000.0
PEAK_FLOPS = {"bf16": 2.5e15, "fp32": 157.3e12}


def load_shape(index=2):
    """Layer sizes of a benchmark configuration, from BASELINE.json's configs[index]. Every
    field must be found where the sentence is expected to give it; a reworded sentence raises
    rather than yield another model."""
    import re
    with open(os.path.join(ROOT, "BASELINE.json")) as f:
        text = json.load(f)["configs"][index]

    def find(field, pattern, convert=int):
        found = re.findall(pattern, text)
        if len(found) != 1:
            raise ValueError(f"BASELINE.json configs[{index}]: expected {field} once as /{pattern}/, "
                             f"found {found!r} in: {text!r}")
        return convert(found[0])

    tied, separate = "tied embeddings" in text, "separate lm_head" in text
    if tied == separate:
        raise ValueError(f"BASELINE.json configs[{index}]: neither or both of 'tied embeddings' and "
                         f"'separate lm_head' in: {text!r}")
    shape = dict(
        num_hidden_layers=find("layers", r"Model: (\d+) layers"), hidden_size=find("hidden", r"hidden (\d+),"),
        num_attention_heads=find("query heads", r"(\d+) query heads"),
        num_key_value_heads=find("KV heads", r"(\d+) KV heads"),
        head_dim=find("head_dim", r"head_dim (\d+)[, ]"), intermediate_size=find("intermediate", r"intermediate (\d+),"),
        vocab_size=find("vocab", r"vocab (\d+),"), rope_theta=find("rope_theta", r"rope_theta ([0-9.e+]+),", float),
        rms_norm_eps=find("rms_norm_eps", r"rms_norm_eps ([0-9.e-]+),", float), tie_word_embeddings=tied)
    shape["context"] = find("context length", r"Context length (\d+) per sequence") if index == 2 else 0
    for key, value in shape.items():
        if key not in ("tie_word_embeddings", "context") and not value > 0:
            raise ValueError(f"BASELINE.json configs[{index}]: {key} = {value}")
    return shape


def workload_bytes(cfg, layers, elem):
    """(bytes of weights a decode step reads once, bytes of cache per token held)."""
    H, I, V = cfg.hidden_size, cfg.intermediate_size, cfg.vocab_size
    per_layer = (cfg.q_dim + 2 * cfg.kv_dim) * H + H * cfg.q_dim + 3 * H * I
    return (layers * per_layer + V * H) * elem, layers * 2 * cfg.kv_dim * elem, per_layer


def run_workload(args, index, new=None):
    """The other two workloads of the benchmark description, through the generation loop:
    configs[3] (1.7B shape: 16 prompts of 64..1024 tokens, 256 new tokens each) and configs[4]
    (32B shape: 8 prompts of 2048 tokens, 512 new tokens each). Returns the record as a dict."""
    import torch
    import herbert_rs_amd as hb
    from herbert_rs_amd.sampling import SamplingParams
    shape = load_shape(index)
    shape.pop("context")
    layers_full = shape["num_hidden_layers"]
    if args.layers:
        shape["num_hidden_layers"] = args.layers
    gen = torch.Generator().manual_seed(index)
    if index == 3:
        lengths = torch.randint(64, 1025, (16,), generator=gen).tolist()
        default_new, name = 256, "Qwen3-1.7B shape"
    else:
        lengths, default_new, name = [2048] * 8, 512, "Qwen3-32B shape"
    new = new or default_new
    raw = dict(shape, architectures=["Qwen3ForCausalLM"], model_type="qwen3",
               max_position_embeddings=4096, eos_token_id=151645)
    cfg = hb.Qwen3Config.from_dict(raw)
    torch.cuda.set_device(0)
    t0 = time.time()
    room = sum((n + new + 127) // 64 * 64 for n in lengths)
    engine = hb.Engine.from_config(cfg, seed=index, dtype=args.dtype, max_tokens=room, max_slots=len(lengths))
    print(f"[bench] {name} built in {time.time() - t0:.1f} s", file=sys.stderr, flush=True)
    prompts = [torch.randint(0, cfg.vocab_size, (n,), generator=gen).tolist() for n in lengths]
    params = SamplingParams(temperature=0.0, max_tokens=new, ignore_eos=True, repeat_check=False)
    engine.generate(prompts[:2], SamplingParams(temperature=0.0, max_tokens=3, ignore_eos=True,
                                                repeat_check=False))              # compiles, warms
    results = engine.generate(prompts, params, max_batch=len(prompts))
    st = engine.last_generation_stats
    assert all(len(r.tokens) == new for r in results)
    decoded = st.generated_tokens - len(prompts)
    ms = st.decode_seconds / st.decode_steps * 1e3
    elem = 2 if args.dtype == "bfloat16" else 4
    weight_bytes, kv_per_token, _ = workload_bytes(cfg, cfg.num_hidden_layers, elem)
    held = sum(n + new / 2.0 for n in lengths)          # tokens in the cache at the middle of the decode
    gbs = (weight_bytes + held * kv_per_token) / (ms * 1e-3) / 1e9
    del engine
    torch.cuda.empty_cache()
    return {
        "metric": f"decode tok/s, {name}, batch {len(prompts)}, {new} new tokens each",
        "value": round(decoded / st.decode_seconds, 2), "unit": "tokens/s", "n_gpus": 1,
        "steps": st.decode_steps, "warmup": 0, "ms_per_step": round(ms, 4),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16" if args.dtype == "bfloat16" else "fp32",
        "data": "synthetic: random weights of standard deviation 0.02 (near normal: sums of eight random bytes), random token ids",
        "config": {"model": name, "layers": layers_full, "layers_run": cfg.num_hidden_layers,
                   "hidden_size": cfg.hidden_size,
                   "num_attention_heads": cfg.num_attention_heads,
                   "num_key_value_heads": cfg.num_key_value_heads, "head_dim": cfg.head_dim,
                   "intermediate_size": cfg.intermediate_size, "vocab_size": cfg.vocab_size,
                   "tie_word_embeddings": cfg.tie_word_embeddings, "global_batch": len(prompts),
                   "prompt_tokens": st.prompt_tokens, "new_tokens": new, "parallelism": "single GPU"},
        "prefill": {"value": round(st.prompt_tokens / st.prefill_seconds, 1), "tokens": st.prompt_tokens,
                    "ms": round(st.prefill_seconds * 1e3, 3)},
        "roofline": {"bound": "hbm", "achieved": round(gbs, 1), "peak": HBM_GBS, "unit": "GB/s",
                     "frac": round(gbs / HBM_GBS, 4)},
    }


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=32)
    ap.add_argument("--warmup", type=int, default=4)
    ap.add_argument("--layers", type=int, default=None, help="run fewer layers than the configuration has")
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--context", type=int, default=None)
    ap.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    ap.add_argument("--no-points", action="store_true", help="skip batch 1 and 64 and the prefill")
    ap.add_argument("--no-workloads", action="store_true",
                    help="skip the 1.7B and 32B workloads that the default run adds to `points`")
    ap.add_argument("--no-sweep", action="store_true", help="time the full context only, not 512 and the mean")
    ap.add_argument("--no-long", action="store_true",
                    help="skip the further sizes and lengths (contexts of 16 K and 32 K, batch 128 and 256, long prompts)")
    ap.add_argument("--workload", default="headline", choices=["headline", "qwen3-1.7b", "qwen3-32b"],
                    help="headline: BASELINE.json configs[2]; the others: configs[3] and configs[4]")
    ap.add_argument("--prefill-tokens", type=int, default=2048, help="length of the prompt of the prefill figure")
    ap.add_argument("--prefill-chunk", type=int, default=0,
                    help="feed the prompt of the prefill figure in steps of this many tokens (0: in one step)")
    ap.add_argument("--prefill-only", action="store_true",
                    help="run the 2,048-token prefill alone (for profiles); prints no JSON line")
    ap.add_argument("--temperature", type=float, default=0.0,
                    help="choose the decode steps' tokens by sampling at this temperature (top-k 40, top-p 0.9) "
                         "instead of argmax")
    ap.add_argument("--contexts", default=None,
                    help="decode one batch whose sequences hold these numbers of tokens (comma-separated, "
                         "e.g. 32768,1024,1024: unequal lengths); prints ms a step and GB/s, no JSON line")
    args = ap.parse_args()
    if args.gpus != 1:
        print(f"bench.py measures one GPU only: --gpus {args.gpus} is not supported (this library "
              "does no work on several GPUs)")
        return 2

    if args.workload != "headline":
        print(json.dumps(run_workload(args, 3 if args.workload == "qwen3-1.7b" else 4,
                                      new=None if args.steps == 32 else args.steps)))
        return 0

    import torch
    import herbert_rs_amd as hb
    from herbert_rs_amd.engine import StepEntry
    from herbert_rs_amd.sampling import SamplingParams
    from herbert_rs_amd.sampling.sampler import Sampler

    shape = load_shape()
    unequal = [int(c) for c in args.contexts.split(",")] if args.contexts else None
    if unequal:
        args.context, args.batch, args.no_points = max(unequal), len(unequal), True
    context = args.context or shape.pop("context")
    shape.pop("context", None)
    layers_full = shape["num_hidden_layers"]
    layers = args.layers or layers_full
    long_points = not (args.no_points or args.no_long or unequal or args.prefill_only)
    LONG_CONTEXTS, LONG_BATCHES, LONG_PROMPTS, LONG_CHUNK = (16384, 32768), (128, 256), (8192, 16384, 32768), 8192
    longest = max(LONG_CONTEXTS + LONG_PROMPTS) if long_points else 0
    raw = dict(shape, architectures=["Qwen3ForCausalLM"], model_type="qwen3",
               num_hidden_layers=layers, max_position_embeddings=max(context, 4096, args.prefill_tokens, longest) + 64,
               eos_token_id=151645)
    cfg = hb.Qwen3Config.from_dict(raw)
    torch.cuda.set_device(0)
    max_batch = args.batch if args.no_points else max(args.batch, 64)
    cache_tokens = max(max_batch * (context + 64), args.prefill_tokens + 64)
    if long_points:
        max_batch = max(max_batch, max(LONG_BATCHES))
        cache_tokens = max(cache_tokens, max(LONG_BATCHES) * (context + 64), 64 * (LONG_CONTEXTS[0] + 64),
                           args.batch * (LONG_CONTEXTS[1] + 64))
    if unequal:
        cache_tokens = sum((c + 127) // 64 * 64 for c in unequal)
    t0 = time.time()
    engine = hb.Engine.from_config(cfg, seed=2, dtype=args.dtype, std=0.02, norm_std=0.0,
                                   max_tokens=cache_tokens, max_slots=max_batch)
    print(f"[bench] model built in {time.time() - t0:.1f} s", file=sys.stderr, flush=True)
    gen = torch.Generator().manual_seed(5)
    elem = 2 if args.dtype == "bfloat16" else 4

    def ids(n):
        return torch.randint(0, cfg.vocab_size, (n,), generator=gen).tolist()

    # bytes of weights that one decode step reads once
    H, I, V = cfg.hidden_size, cfg.intermediate_size, cfg.vocab_size
    weight_bytes, kv_bytes_per_token, per_layer = workload_bytes(cfg, layers, elem)

    headline_params = SamplingParams(temperature=0.0) if args.temperature <= 0 else \
        SamplingParams(temperature=args.temperature, top_k=40, top_p=0.9, seed=1)

    def step_gbs(batch, mean_context, ms):
        return (weight_bytes + batch * mean_context * kv_bytes_per_token) / (ms * 1e-3) / 1e9

    def decode_run(batch, plan, run_ahead=True, fill_chunk=2048, params=None):
        """[(context, tokens/s, ms/step)] for each (context, steps, warmup) of `plan` (contexts
        ascending): `steps` timed decode steps at `batch` after `warmup` untimed ones, ending with
        every sequence holding `context` tokens; one pass over a cache that is filled by real
        prefill of random prompts up to where each run's steps begin."""
        slots = [engine.alloc_slot() for _ in range(batch)]
        chooser = Sampler(params or headline_params, batch, V, engine.device)
        tokens = [ids(1)[0] for _ in range(batch)]
        held, chunk, out = 0, fill_chunk, []

        ahead = [None]

        def one():
            """A decode step as the generation loop runs it: put on the stream with the tokens of the
            step before still on the GPU, whose copy the host reads while this step runs."""
            if not run_ahead:       # the host reads a step's tokens before it starts the next
                logits = engine.step([StepEntry(s, [t], [0]) for s, t in zip(slots, tokens)], keep_logits=False)
                return chooser.choose(logits, range(batch))
            before = ahead[0]
            if before is None:
                logits = engine.step([StepEntry(s, [t], [0]) for s, t in zip(slots, tokens)], keep_logits=False)
            else:
                logits = engine.step([StepEntry(s, [0], [0]) for s in slots], tokens_on_device=before.device, keep_logits=False)
            ahead[0] = chooser.choose_ahead(logits, range(batch))
            return tokens if before is None else chooser.read(before)
        for c, steps, warmup in plan:
            fill = c - steps - warmup - held
            if fill < 0:
                raise ValueError(f"context {c} leaves no room for {steps} + {warmup} steps after {held} tokens")
            for s in slots:
                for a in range(0, fill, chunk):
                    engine.step([StepEntry(s, ids(min(chunk, fill - a)), [])])
            for _ in range(warmup):
                tokens = one()
            torch.cuda.synchronize()
            t = time.perf_counter()
            for _ in range(steps):
                tokens = one()
            torch.cuda.synchronize()
            dt = time.perf_counter() - t
            held = c
            out.append((c, batch * steps / dt, dt / steps * 1e3))
        for s in slots:
            engine.free_slot(s)
        return out

    def prefill_once(tokens_n, chunk=None):
        """One prompt of tokens_n tokens, whole or in chunks; the last token's logits are asked for."""
        slot = engine.alloc_slot()
        chunk = chunk or args.prefill_chunk or tokens_n
        prompt = ids(tokens_n)
        for a in range(0, tokens_n, chunk):
            part = prompt[a:a + chunk]
            engine.step([StepEntry(slot, part, [len(part) - 1] if a + chunk >= tokens_n else [])])
        engine.free_slot(slot)

    def prefill_run(tokens_n, reps, chunk=None, warm=True):
        if warm:
            prefill_once(tokens_n, chunk)
        torch.cuda.synchronize()
        t = time.perf_counter()
        for _ in range(reps):
            prefill_once(tokens_n, chunk)
        torch.cuda.synchronize()
        return (time.perf_counter() - t) / reps

    def prefill_flops(T):
        return 2.0 * T * (layers * per_layer) + 2.0 * V * H + layers * 4.0 * cfg.q_dim * T * (T + 1) / 2.0

    def unequal_run(contexts, steps, warmup):
        """(ms a step, GB/s) of one batch whose sequences hold `contexts` tokens after the timed
        steps, decoded as the generation loop does (each step put on the stream one ahead)."""
        if min(contexts) <= steps + warmup:
            raise ValueError(f"every sequence of {contexts} needs more than {steps + warmup} tokens")
        slots = [engine.alloc_slot() for _ in contexts]
        for s, c in zip(slots, contexts):
            fill = c - steps - warmup
            for a in range(0, fill, 2048):
                engine.step([StepEntry(s, ids(min(2048, fill - a)), [])])
        chooser = Sampler(SamplingParams(temperature=0.0), len(slots), V, engine.device)
        ahead = chooser.choose_ahead(engine.step([StepEntry(s, ids(1), [0]) for s in slots], keep_logits=False), range(len(slots)))
        for n in (warmup - 1, steps):
            torch.cuda.synchronize()
            t = time.perf_counter()
            for _ in range(n):
                logits = engine.step([StepEntry(s, [0], [0]) for s in slots], tokens_on_device=ahead.device, keep_logits=False)
                before, ahead = ahead, chooser.choose_ahead(logits, range(len(slots)))
                chooser.read(before)
            torch.cuda.synchronize()
            ms = (time.perf_counter() - t) / max(1, n) * 1e3
        for s in slots:
            engine.free_slot(s)
        held = sum(contexts) - len(contexts) * steps / 2.0
        return ms, (weight_bytes + held * kv_bytes_per_token) / (ms * 1e-3) / 1e9, held

    if unequal:
        ms, gbs, held = unequal_run(unequal, args.steps, max(2, args.warmup))
        print(f"[bench] decode of {len(unequal)} sequences holding {args.contexts} tokens: {ms:.3f} ms a step, "
              f"{len(unequal) / ms * 1e3:.0f} tok/s, {gbs:.0f} GB/s of {HBM_GBS:.0f} "
              f"(weights {weight_bytes / 1e9:.2f} GB + keys and values {held * kv_bytes_per_token / 1e9:.2f} GB)",
              file=sys.stderr, flush=True)
        return 0
    if args.prefill_only:
        sec = prefill_run(args.prefill_tokens, max(1, args.steps))
        print(f"[bench] prefill {args.prefill_tokens}: {args.prefill_tokens / sec:.0f} tok/s, {sec * 1e3:.2f} ms",
              file=sys.stderr, flush=True)
        return 0
    # contexts of the sweep: 512 (where the described decode starts), the full context, and a
    # few in between for the mean over a decode from the one to the other
    sweep_steps, sweep_warmup = min(args.steps, 12), 3
    low = 512
    between = [] if args.no_sweep or args.no_points or context <= low + 64 else \
        [c for c in (low, 1024, 2048, 3072) if c < context - args.steps - args.warmup - sweep_steps]

    def measure(batch):
        """(at the full context, at 512 or None, mean over 512 -> full context or None), each
        (tokens/s, ms/step, GB/s)."""
        # the sweep's shorter runs first, in one pass over a cache that grows; the full context is
        # timed with exactly --steps steps after --warmup
        runs = decode_run(batch, [(c, sweep_steps, sweep_warmup) for c in between]
                          + [(context, args.steps, args.warmup)])
        full = runs.pop()
        at_full = (full[1], full[2], step_gbs(batch, context - args.steps / 2.0, full[2]))
        if not runs:
            return at_full, None, None
        c0, v0, ms0 = runs[0]
        at_low = (v0, ms0, step_gbs(batch, c0 - sweep_steps / 2.0, ms0))
        pts = [(c - sweep_steps / 2.0, ms_c) for c, _, ms_c in runs] + [(context - args.steps / 2.0, full[2])]
        area = sum((pts[i + 1][0] - pts[i][0]) * (pts[i + 1][1] + pts[i][1]) / 2.0 for i in range(len(pts) - 1))
        mean_ms = area / (pts[-1][0] - pts[0][0])
        mean_ctx = (pts[-1][0] + pts[0][0]) / 2.0
        return at_full, at_low, (batch / mean_ms * 1e3, mean_ms, step_gbs(batch, mean_ctx, mean_ms))

    def add_points(points, batch, result):
        at_full, at_low, mean = result
        for tag, r in (("", at_full), ("_ctx512", at_low), ("_mean_512_to_full", mean)):
            if r is None:
                continue
            key = f"decode_b{batch}{tag}"
            points[key] = round(r[0], 2)
            points[key + "_ms"] = round(r[1], 4)
            points[key + "_gbs"] = round(r[2], 1)
            points[key + "_frac"] = round(r[2] / HBM_GBS, 4)

    points = {}
    head = measure(args.batch)
    value, ms, achieved = head[0]
    add_points(points, args.batch, head)
    if not args.no_points:
        # for comparison: the same step with the host between two steps (it reads a step's tokens,
        # then starts the next), as the loop runs where a sampler's choice needs the host
        _, v_sync, ms_sync = decode_run(args.batch, [(context, min(args.steps, 16), 3)], run_ahead=False)[0]
        points[f"decode_b{args.batch}_host_between_steps"] = round(v_sync, 2)
        points[f"decode_b{args.batch}_host_between_steps_ms"] = round(ms_sync, 4)
        # and with the command line's default sampling (temperature 0.4, top-k 40, top-p 0.9) in place of argmax
        _, v_drawn, ms_drawn = decode_run(args.batch, [(context, min(args.steps, 16), 3)],
                                          params=SamplingParams(temperature=0.4, top_k=40, top_p=0.9, seed=1))[0]
        points[f"decode_b{args.batch}_sampled"] = round(v_drawn, 2)
        points[f"decode_b{args.batch}_sampled_ms"] = round(ms_drawn, 4)
        # a batch of unequal lengths: one sequence at the full context beside fifteen of a sixteenth
        mixed = [context] + [max(context // 16, 64)] * 15
        ms_mixed, gbs_mixed, _ = unequal_run(mixed, min(args.steps, 16), 3)
        points["decode_b16_unequal_lengths_ms"] = round(ms_mixed, 4)
        points["decode_b16_unequal_lengths"] = round(len(mixed) / ms_mixed * 1e3, 2)
        points["decode_b16_unequal_lengths_gbs"] = round(gbs_mixed, 1)
    for key in (f"decode_b{args.batch}", f"decode_b{args.batch}_ms", f"decode_b{args.batch}_gbs",
                f"decode_b{args.batch}_frac"):
        points.pop(key)          # the headline itself: `value`, `ms_per_step`, `roofline`
    out = {
        "metric": "decode tok/s at batch 8, Qwen3-8B shape, context 4096 (+ prefill tok/s at 2048 "
                  "tokens, decode at batch 1 and 64)" + (f", tokens sampled at temperature {args.temperature}"
                                                         if args.temperature > 0 else ""),
        "value": round(value, 2), "unit": "tokens/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": round(ms, 4), "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16" if args.dtype == "bfloat16" else "fp32",
        "data": "synthetic: random weights of standard deviation 0.02 (near normal: sums of eight random bytes), "
                "random token ids, cache filled by prefill of random prompts",
        "config": {
            "model": "Qwen3-8B shape", "layers": layers_full, "layers_run": layers,
            "hidden_size": H, "num_attention_heads": cfg.num_attention_heads,
            "num_key_value_heads": cfg.num_key_value_heads, "head_dim": cfg.head_dim,
            "intermediate_size": I, "vocab_size": V, "rope_theta": cfg.rope_theta,
            "rms_norm_eps": cfg.rms_norm_eps, "tie_word_embeddings": cfg.tie_word_embeddings,
            "global_batch": args.batch, "seq_len": context, "prefill_tokens": args.prefill_tokens,
            "parallelism": "single GPU",
        },
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_GBS, "unit": "GB/s",
                     "frac": round(achieved / HBM_GBS, 4)},
    }
    if not args.no_points:
        T = args.prefill_tokens
        sec = prefill_run(T, 5)
        peak = PEAK_FLOPS["bf16" if args.dtype == "bfloat16" else "fp32"]
        out["prefill"] = {"value": round(T / sec, 1), "tokens": T, "ms": round(sec * 1e3, 3),
                          "frac": round(prefill_flops(T) / sec / peak, 4)}
        print(f"[bench] prefill {T}: {T / sec:.0f} tok/s", file=sys.stderr, flush=True)
        for batch in (1, 64):
            if batch != args.batch:
                r = measure(batch)
                add_points(points, batch, r)
                print(f"[bench] decode b{batch}: {r[0][0]:.1f} tok/s, {r[0][1]:.3f} ms/step", file=sys.stderr, flush=True)
        if long_points:
            # further sizes and lengths, each in one pass over a cache filled by prefill in chunks
            for T in LONG_PROMPTS:
                sec = prefill_run(T, 2 if T <= 16384 else 1, chunk=LONG_CHUNK, warm=T == LONG_PROMPTS[0])
                points[f"prefill_{T}"] = round(T / sec, 1)
                points[f"prefill_{T}_frac"] = round(prefill_flops(T) / sec / peak, 4)
                print(f"[bench] prefill {T} in chunks of {LONG_CHUNK}: {T / sec:.0f} tok/s", file=sys.stderr, flush=True)
            few = min(args.steps, 12)

            def add_long(batch, runs, label):
                for c, v, ms_c in runs:
                    key = f"decode_b{batch}" + (f"_ctx{c}" if label else "")
                    gbs = step_gbs(batch, c - few / 2.0, ms_c)
                    points[key], points[key + "_ms"] = round(v, 2), round(ms_c, 4)
                    points[key + "_gbs"], points[key + "_frac"] = round(gbs, 1), round(gbs / HBM_GBS, 4)
                    print(f"[bench] decode b{batch} at {c} tokens: {v:.1f} tok/s, {ms_c:.3f} ms/step", file=sys.stderr,
                          flush=True)
            add_long(args.batch, decode_run(args.batch, [(c, few, 3) for c in LONG_CONTEXTS], fill_chunk=LONG_CHUNK), True)
            add_long(64, decode_run(64, [(LONG_CONTEXTS[0], few, 3)], fill_chunk=LONG_CHUNK), True)
            for batch in LONG_BATCHES:
                add_long(batch, decode_run(batch, [(context, few, 3)], fill_chunk=2048), False)
        if not args.no_workloads and not args.layers:
            del engine
            torch.cuda.empty_cache()
            for index, tag in ((3, "qwen3_1p7b_b16"), (4, "qwen3_32b_b8")):
                rec = run_workload(args, index)
                points[tag + "_decode"] = rec["value"]
                points[tag + "_decode_ms"] = rec["ms_per_step"]
                points[tag + "_decode_gbs"] = rec["roofline"]["achieved"]
                points[tag + "_decode_frac"] = rec["roofline"]["frac"]
                points[tag + "_prefill"] = rec["prefill"]["value"]
                print(f"[bench] {rec['config']['model']}: {rec['value']:.1f} tok/s, {rec['ms_per_step']:.3f} ms/step",
                      file=sys.stderr, flush=True)
    if points:
        out["points"] = points
    print(json.dumps(out))
    return 0


if __name__ == "__main__":
    sys.exit(main())
