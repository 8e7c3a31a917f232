"""Command line in the manner of the reference's herbert-cli (crates/cli/src/main.rs:54-195).

Kept with their names, meanings and defaults: --model, --prompt, --prompt-file, --system,
--max-tokens (2048), --ignore-eos, --no-repeat-check, --stop, --verbose, --temperature (0.4,
0 = greedy), --top-k (40, 0 = off), --top-p (0.9, 1.0 = off), --show-specials. Added here:
--dtype, --seed, --cache-tokens, and --random-weights to write a random model folder.
With a tokenizer.json in the model folder the prompt is text wrapped in the ChatML
template (main.rs:281-294); without one it is comma-separated token ids
(crates/cli/src/token_parser.rs:13-26) and the output is token ids.
"""
import argparse
import json
import os
import sys
import time

from .errors import HerbertError, RequestError


def build_prompt(user_prompt, system_prompt=None):
    """ChatML as the reference builds it for this family (crates/cli/src/main.rs:281-294)."""
    out = ""
    if system_prompt:
        out += "<|im_start|>system\n" + system_prompt + "<|im_end|>\n"
    out += "<|im_start|>user\n" + user_prompt + "<|im_end|>\n<|im_start|>assistant\n"
    return out


def parse_token_ids(text):
    """Comma-separated token ids (crates/cli/src/token_parser.rs:13-26)."""
    if "," not in text and not text.strip().isdigit():
        raise RequestError("Need tokenizer.json or comma-separated token IDs")
    ids = []
    for piece in text.split(","):
        piece = piece.strip()
        if not piece.isdigit():
            raise RequestError(f"Invalid token ID '{piece}'")
        ids.append(int(piece))
    return ids


def load_tokenizer(model_dir):
    path = os.path.join(model_dir, "tokenizer.json")
    if not os.path.exists(path):
        return None
    from tokenizers import Tokenizer
    return Tokenizer.from_file(path)


def make_parser():
    ap = argparse.ArgumentParser(prog="herbert-cli", description="Herbert - local LLM inference on MI355X")
    ap.add_argument("--model", required=True, help="Model directory")
    ap.add_argument("--prompt", help="Input prompt (text with a tokenizer, else comma-separated ids)")
    ap.add_argument("--prompt-file", help="Read prompt from a file")
    ap.add_argument("--system", help="System prompt (prepended with chat template)")
    ap.add_argument("--max-tokens", type=int, default=2048, help="Max tokens to generate")
    ap.add_argument("--ignore-eos", action="store_true", help="Ignore EOS token")
    ap.add_argument("--no-repeat-check", action="store_true", help="Disable repetition loop detection")
    ap.add_argument("--stop", action="append", default=[],
                    help="Stop sequence (repeatable); without a tokenizer a token id")
    ap.add_argument("--verbose", action="store_true", help="Show stats after generation")
    ap.add_argument("--temperature", type=float, default=0.4, help="Sampling temperature (0 = greedy argmax)")
    ap.add_argument("--top-k", type=int, default=40, help="Top-k sampling (0 = disabled)")
    ap.add_argument("--top-p", type=float, default=0.9, help="Top-p / nucleus sampling (1.0 = disabled)")
    ap.add_argument("--show-specials", action="store_true", help="Show special tokens in output")
    ap.add_argument("--seed", type=int, default=None, help="Sampler seed (default: from the clock)")
    ap.add_argument("--dtype", choices=["bfloat16", "float32"], default="bfloat16")
    ap.add_argument("--cache-tokens", type=int, default=None,
                    help="tokens the cache holds (default: prompt + max-tokens)")
    ap.add_argument("--random-weights", action="store_true",
                    help="write random weights for --model's config.json (with --seed) if it has none")
    return ap


def main(argv=None):
    args = make_parser().parse_args(argv)
    try:
        return _run(args)
    except HerbertError as e:
        print(f"herbert-cli: {e}", file=sys.stderr)
        return 1


def _run(args):
    from .api import load, write_random_model
    from .sampling import SamplingParams
    if args.random_weights and not os.path.exists(os.path.join(args.model, "model.safetensors")):
        write_random_model(args.model, os.path.join(args.model, "config.json"), seed=args.seed or 0,
                           dtype=args.dtype)
    prompt = args.prompt
    if args.prompt_file:
        with open(args.prompt_file) as f:
            prompt = f.read()
    if prompt is None:
        raise RequestError("--prompt or --prompt-file is required (there is no interactive mode)")
    tokenizer = load_tokenizer(args.model)
    if tokenizer is not None:
        ids = tokenizer.encode(build_prompt(prompt, args.system), add_special_tokens=False).ids
    else:
        ids = parse_token_ids(prompt)
    stop_ids = []
    stop_strings = []
    for s in args.stop:
        if tokenizer is None:
            stop_ids.extend(parse_token_ids(s))
        else:
            stop_strings.append(s.encode().decode("unicode_escape"))
    if tokenizer is not None:
        im_end = tokenizer.token_to_id("<|im_end|>")
        if im_end is not None:
            stop_ids.append(im_end)

    t0 = time.perf_counter()
    cache_tokens = args.cache_tokens or (len(ids) + args.max_tokens + 64)
    engine = load(args.model, dtype=args.dtype, cache_tokens=cache_tokens)
    load_seconds = time.perf_counter() - t0

    params = SamplingParams(temperature=args.temperature, top_k=args.top_k, top_p=args.top_p,
                            max_tokens=args.max_tokens, stop_ids=tuple(stop_ids),
                            ignore_eos=args.ignore_eos, repeat_check=not args.no_repeat_check,
                            seed=args.seed)
    produced = []
    printed = [0]

    def on_token(_, tok):
        produced.append(tok)
        if tokenizer is None:
            print(tok if len(produced) == 1 else f",{tok}", end="", flush=True)
        else:
            text = tokenizer.decode(produced, skip_special_tokens=not args.show_specials)
            if not text.endswith("�"):
                print(text[printed[0]:], end="", flush=True)
                printed[0] = len(text)

    t0 = time.perf_counter()
    result = engine.generate([ids], params, on_token=on_token)[0]
    total = time.perf_counter() - t0
    print()
    if args.verbose:
        st = engine.last_generation_stats
        decoded = max(0, st.generated_tokens - 1)
        err = sys.stderr
        print("--- Stats ---", file=err)
        print("Backend:         hip-gfx950", file=err)
        print(f"Model load:      {load_seconds:.3f}s", file=err)
        print(f"Input tokens:    {st.prompt_tokens}", file=err)
        print(f"Output tokens:   {st.generated_tokens}", file=err)
        pf = st.prompt_tokens / st.prefill_seconds if st.prefill_seconds > 0 else 0.0
        dc = decoded / st.decode_seconds if st.decode_seconds > 0 else 0.0
        print(f"Prefill:         {st.prefill_seconds:.3f}s ({pf:.1f} tok/s)", file=err)
        print(f"Decode:          {st.decode_seconds:.3f}s ({dc:.1f} tok/s)", file=err)
        print(f"Total:           {total:.3f}s", file=err)
        print(f"Stop reason:     {result.stop_reason}", file=err)
    return 0


if __name__ == "__main__":
    sys.exit(main())
