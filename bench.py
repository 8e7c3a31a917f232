"""Decode and prefill throughput of the Qwen3-8B shape (BASELINE.json configs[2]) on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--layers L] [--batch B] [--context C]

One JSON line: `value` is decoded tokens a second at batch 8 with every sequence holding
`context` tokens; `prefill` is one 2,048-token prompt; `roofline` prices the decode step
against HBM; `points` holds decode at batch 1 and 64. Weights are random, token ids are
random, and the cache below the timed steps is filled by real prefill steps of random prompts.
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
    """Layer sizes of a benchmark configuration, parsed from BASELINE.json's configs[index]."""
    import re
    with open(os.path.join(ROOT, "BASELINE.json")) as f:
        text = json.load(f)["configs"][index]

    def num(pattern):
        return int(re.search(pattern, text).group(1))
    return dict(
        num_hidden_layers=num(r"(\d+) layers"), hidden_size=num(r"hidden (\d+)"),
        num_attention_heads=num(r"(\d+) query heads"), num_key_value_heads=num(r"(\d+) KV heads"),
        head_dim=num(r"head_dim (\d+)"), intermediate_size=num(r"intermediate (\d+)"),
        vocab_size=num(r"vocab (\d+)"),
        context=num(r"Context length (\d+)") if "Context length" in text else 0,
        rope_theta=1e6, rms_norm_eps=1e-6, tie_word_embeddings="tied embeddings" in text)


def run_workload(args, index):
    """The other two workloads of the benchmark description, through the generation loop:
    configs[3] (1.7B shape: 16 prompts of 64..1024 tokens, 256 new tokens each) and configs[4]
    (32B shape: 8 prompts of 2048 tokens, 512 new tokens each)."""
    import torch
    import herbert_rs_amd as hb
    from herbert_rs_amd.sampling import SamplingParams
    shape = load_shape(index)
    shape.pop("context")
    if args.layers:
        shape["num_hidden_layers"] = args.layers
    gen = torch.Generator().manual_seed(index)
    if index == 3:
        lengths = torch.randint(64, 1025, (16,), generator=gen).tolist()
        new, name = 256, "Qwen3-1.7B shape"
    else:
        lengths, new, name = [2048] * 8, 512, "Qwen3-32B shape"
    if args.steps != 32:
        new = args.steps
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
    print(json.dumps({
        "metric": f"decode tok/s, {name}, batch {len(prompts)}, {new} new tokens each",
        "value": round(decoded / st.decode_seconds, 2), "unit": "tokens/s", "n_gpus": 1,
        "steps": st.decode_steps, "warmup": 0, "ms_per_step": round(st.decode_seconds / st.decode_steps * 1e3, 4),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16" if args.dtype == "bfloat16" else "fp32",
        "data": "synthetic: random weights N(0, 0.02), random token ids",
        "config": {"model": name, "layers": cfg.num_hidden_layers, "hidden_size": cfg.hidden_size,
                   "num_attention_heads": cfg.num_attention_heads,
                   "num_key_value_heads": cfg.num_key_value_heads, "head_dim": cfg.head_dim,
                   "intermediate_size": cfg.intermediate_size, "vocab_size": cfg.vocab_size,
                   "tie_word_embeddings": cfg.tie_word_embeddings, "global_batch": len(prompts),
                   "prompt_tokens": st.prompt_tokens, "new_tokens": new, "parallelism": "single GPU"},
        "prefill": {"value": round(st.prompt_tokens / st.prefill_seconds, 1), "tokens": st.prompt_tokens,
                    "ms": round(st.prefill_seconds * 1e3, 3)},
    }))
    return 0


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
    ap.add_argument("--workload", default="headline", choices=["headline", "qwen3-1.7b", "qwen3-32b"],
                    help="headline: BASELINE.json configs[2]; the others: configs[3] and configs[4]")
    ap.add_argument("--prefill-tokens", type=int, default=2048, help="length of the prompt of the prefill figure")
    ap.add_argument("--prefill-only", action="store_true",
                    help="run the 2,048-token prefill alone (for profiles); prints no JSON line")
    args = ap.parse_args()
    if args.gpus != 1:
        print(f"bench.py measures one GPU only: --gpus {args.gpus} is not supported (this library "
              "does no work on several GPUs)")
        return 2

    if args.workload != "headline":
        return run_workload(args, 3 if args.workload == "qwen3-1.7b" else 4)

    import torch
    import herbert_rs_amd as hb
    from herbert_rs_amd.engine import StepEntry
    from herbert_rs_amd.sampling import SamplingParams
    from herbert_rs_amd.sampling.sampler import Sampler

    shape = load_shape()
    context = args.context or shape.pop("context")
    shape.pop("context", None)
    layers_full = shape["num_hidden_layers"]
    layers = args.layers or layers_full
    raw = dict(shape, architectures=["Qwen3ForCausalLM"], model_type="qwen3",
               num_hidden_layers=layers, max_position_embeddings=max(context, 4096) + 64,
               eos_token_id=151645)
    cfg = hb.Qwen3Config.from_dict(raw)
    torch.cuda.set_device(0)
    max_batch = args.batch if args.no_points else max(args.batch, 64)
    cache_tokens = max_batch * (context + 64)
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
    per_layer = (cfg.q_dim + 2 * cfg.kv_dim) * H + H * cfg.q_dim + 3 * H * I
    weight_bytes = (layers * per_layer + V * H) * elem
    kv_bytes_per_token = layers * 2 * cfg.kv_dim * elem

    def decode_run(batch, steps, warmup):
        """tokens/s and ms/step of `steps` decode steps at `batch`, every sequence at `context`."""
        slots = [engine.alloc_slot() for _ in range(batch)]
        fill = context - steps - warmup
        chunk = 2048
        for s in slots:                      # real prefill of random prompts, in chunks
            for a in range(0, fill, chunk):
                n = min(chunk, fill - a)
                engine.step([StepEntry(s, ids(n), [])])
        chooser = Sampler(SamplingParams(temperature=0.0), batch, V, engine.device)
        tokens = [ids(1)[0] for _ in range(batch)]

        def one():
            logits = engine.step([StepEntry(s, [t], [0]) for s, t in zip(slots, tokens)])
            return chooser.choose(logits, range(batch))
        for _ in range(warmup):
            tokens = one()
        torch.cuda.synchronize()
        t = time.perf_counter()
        for _ in range(steps):
            tokens = one()
        torch.cuda.synchronize()
        dt = time.perf_counter() - t
        for s in slots:
            engine.free_slot(s)
        return batch * steps / dt, dt / steps * 1e3

    def prefill_run(tokens_n, reps):
        slot = engine.alloc_slot()
        engine.step([StepEntry(slot, ids(tokens_n), [tokens_n - 1])])
        engine.free_slot(slot)
        torch.cuda.synchronize()
        t = time.perf_counter()
        for _ in range(reps):
            slot = engine.alloc_slot()
            engine.step([StepEntry(slot, ids(tokens_n), [tokens_n - 1])])
            engine.free_slot(slot)
        torch.cuda.synchronize()
        return (time.perf_counter() - t) / reps

    if args.prefill_only:
        sec = prefill_run(args.prefill_tokens, max(1, args.steps))
        print(f"[bench] prefill {args.prefill_tokens}: {args.prefill_tokens / sec:.0f} tok/s, {sec * 1e3:.2f} ms",
              file=sys.stderr, flush=True)
        return 0
    value, ms = decode_run(args.batch, args.steps, args.warmup)
    print(f"[bench] decode b{args.batch}: {value:.1f} tok/s, {ms:.3f} ms/step", file=sys.stderr, flush=True)
    avg_ctx = context - args.steps / 2.0
    step_bytes = weight_bytes + args.batch * avg_ctx * kv_bytes_per_token
    achieved = step_bytes / (ms * 1e-3) / 1e9
    out = {
        "metric": "decode tok/s at batch 8, Qwen3-8B shape, context 4096 (+ prefill tok/s at 2048 "
                  "tokens, decode at batch 1 and 64)",
        "value": round(value, 2), "unit": "tokens/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": round(ms, 4), "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16" if args.dtype == "bfloat16" else "fp32",
        "data": "synthetic: random weights N(0, 0.02), random token ids, cache filled by prefill of "
                "random prompts",
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
        flops = 2.0 * T * (layers * per_layer) + 2.0 * V * H \
            + layers * 4.0 * cfg.q_dim * T * (T + 1) / 2.0
        peak = PEAK_FLOPS["bf16" if args.dtype == "bfloat16" else "fp32"]
        out["prefill"] = {"value": round(T / sec, 1), "tokens": T, "ms": round(sec * 1e3, 3),
                          "frac": round(flops / sec / peak, 4)}
        print(f"[bench] prefill {T}: {T / sec:.0f} tok/s", file=sys.stderr, flush=True)
        b1, _ = decode_run(1, args.steps, args.warmup)
        print(f"[bench] decode b1: {b1:.1f} tok/s", file=sys.stderr, flush=True)
        b64, _ = decode_run(64, args.steps, args.warmup)
        print(f"[bench] decode b64: {b64:.1f} tok/s", file=sys.stderr, flush=True)
        out["points"] = {"decode_b1": round(b1, 2), "decode_b64": round(b64, 2)}
    print(json.dumps(out))
    return 0


if __name__ == "__main__":
    sys.exit(main())
