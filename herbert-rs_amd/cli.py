"""Command line in the manner of the reference's herbert-cli (crates/cli/src/main.rs:54-195).

Kept with their names, meanings and defaults: --model, --prompt, --prompt-file, --system,
--max-tokens (2048), --ignore-eos, --no-repeat-check, --stop, --verbose, --temperature (0.4,
0 = greedy), --top-k (40, 0 = off), --top-p (0.9, 1.0 = off), --show-specials, --backend (one
backend here; `help` lists it) and --gpu (an index, or `list`). Added here:
--dtype, --seed, --cache-tokens, and --random-weights to write a random model folder.
With a tokenizer.json in the model folder the prompt is text wrapped in the architecture's
chat template (for this family ChatML, main.rs:281-294; the template and the end-of-turn
token are data of the architecture's registry entry); without one it is comma-separated
token ids (crates/cli/src/token_parser.rs:13-26) and the output is token ids.
--stop with a tokenizer is a stop string, matched on the decoded text after every token
(main.rs:236-247,1328-1332,1360); without one it is a token id. --max-tokens counts decode
steps after the token that the prompt gives, as the reference's single shot counts them
(main.rs:1040,1241): up to max-tokens + 1 tokens come out. SIGINT, SIGTERM and SIGHUP set a
flag that the generation loop looks at before every decode step; a second signal exits at
once with 130 (main.rs:22-50,1242-1245). Without --prompt and --prompt-file the conversation
of `chat.py` starts (main.rs:70,718-757), which needs a tokenizer.
"""
import argparse
import os
import signal
import sys
import time

from .errors import HerbertError, RequestError


def decode_escaped_text(raw):
    """\\n, \\r, \\t, \\0 and \\\\ become the characters they name; any other backslash stays
    (crates/cli/src/main.rs:212-234)."""
    out = []
    it = iter(raw)
    for c in it:
        if c != "\\":
            out.append(c)
            continue
        nxt = next(it, None)
        if nxt is None:
            out.append("\\")
        elif nxt in "nrt0\\":
            out.append({"n": "\n", "r": "\r", "t": "\t", "0": "\0", "\\": "\\"}[nxt])
        else:
            out.append("\\" + nxt)
    return "".join(out)


def normalize_stop_sequences(raw):
    """Trimmed, unescaped, without empty ones and repeats (crates/cli/src/main.rs:249-258)."""
    out = []
    for seq in raw:
        decoded = decode_escaped_text(seq.strip())
        if decoded and decoded not in out:
            out.append(decoded)
    return out


def find_stop_sequence(text, stop_sequences):
    """The first stop sequence that the tail of `text` holds, else None: only the last
    (longest stop sequence + 64) bytes are searched (crates/cli/src/main.rs:236-247)."""
    longest = max((len(s.encode()) for s in stop_sequences), default=0)
    tail = text.encode()[-(longest + 64):].decode(errors="ignore") if text else ""
    for seq in stop_sequences:
        if seq in tail:
            return seq
    return None


BACKEND = "hip-gfx950"


class InterruptFlag:
    """Set by the first SIGINT / SIGTERM / SIGHUP; the second exits at once with 130
    (crates/cli/src/main.rs:22-50)."""

    def __init__(self):
        self.count = 0
        self._old = {}

    def __call__(self):
        return self.count > 0

    def _handle(self, signum, frame):
        self.count += 1
        if self.count >= 2:
            os._exit(130)

    def install(self):
        for name in ("SIGINT", "SIGTERM", "SIGHUP"):
            sig = getattr(signal, name, None)
            if sig is not None:
                try:
                    self._old[sig] = signal.signal(sig, self._handle)
                except ValueError:       # not the main thread: the flag can still be set by hand
                    pass
        return self

    def restore(self):
        for sig, old in self._old.items():
            signal.signal(sig, old)
        self._old = {}


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


def print_arch():
    """What --arch shows: the reference prints the CPU's features there (crates/cli/src/arch.rs);
    here it is the GPU the kernels are built for and the one that is present."""
    import torch
    print("herbert-cli: kernels for gfx950 (MI355X), wave64, MFMA bf16")
    if not torch.cuda.is_available():
        print("no GPU visible to this process")
        return 0
    for i in range(torch.cuda.device_count()):
        p = torch.cuda.get_device_properties(i)
        print(f"GPU {i}: {p.name} ({getattr(p, 'gcnArchName', '?')}), {p.multi_processor_count} CUs, "
              f"{p.total_memory / 2**30:.0f} GiB")
    return 0


class StreamPrinter:
    """Prints a sequence's text as its tokens come: the whole text is decoded again each time and
    only what is new is printed, never a trailing U+FFFD, which a later token may still
    complete (crates/cli/src/main.rs:1306-1326). `on_token` is the generation loop's callback;
    it ends the sequence where the text holds a stop string."""

    def __init__(self, tokenizer, show_specials=False, stop_strings=(), out=None):
        self.tokenizer, self.show_specials, self.stop_strings = tokenizer, show_specials, list(stop_strings)
        self.out = out if out is not None else sys.stdout
        self.produced, self.printed = [], 0

    def on_token(self, _, tok):
        from .sampling import STOP_SEQUENCE
        self.produced.append(tok)
        if self.tokenizer is None:
            print(tok if len(self.produced) == 1 else f",{tok}", end="", flush=True, file=self.out)
            return None
        text = self.tokenizer.decode(self.produced, skip_special_tokens=not self.show_specials)
        safe = len(text.rstrip("\ufffd"))
        if safe > self.printed:
            print(text[self.printed:safe], end="", flush=True, file=self.out)
            self.printed = safe
        if self.stop_strings and find_stop_sequence(text, self.stop_strings) is not None:
            return STOP_SEQUENCE
        return None


def end_of_turn_id(chat, tokenizer):
    """The id of the token that ends the model's turn: the tokenizer's, else the architecture's
    own (crates/cli/src/main.rs:616-619); None where the architecture names none."""
    if chat is None or chat.end_of_turn is None:
        return None
    found = tokenizer.token_to_id(chat.end_of_turn) if tokenizer is not None else None
    return found if found is not None else chat.end_of_turn_id


def think_tokens_of(chat, tokenizer):
    """The ids that open and close a think block and of a line break: from the tokenizer, else
    from the architecture's entry (crates/cli/src/main.rs:671-684)."""
    from .sampling import ThinkTokens
    if chat is None or chat.think_open_id is None or chat.think_close_id is None or chat.newline_id is None:
        raise RequestError("--think-budget / --nothink: this architecture names no think tokens")
    open_id, close_id, newline_id = chat.think_open_id, chat.think_close_id, chat.newline_id
    if tokenizer is not None:
        found = tokenizer.token_to_id(chat.think_open)
        open_id = found if found is not None else open_id
        found = tokenizer.token_to_id(chat.think_close)
        close_id = found if found is not None else close_id
        line = tokenizer.encode("\n", add_special_tokens=False).ids
        newline_id = line[0] if len(line) == 1 else newline_id
    return ThinkTokens(open_id, close_id, newline_id)


def check_think_tokens(think_tokens, vocab):
    if think_tokens is not None and not all(0 <= t < vocab for t in (think_tokens.open_id, think_tokens.close_id,
                                                                     think_tokens.newline_id)):
        raise RequestError(f"--think-budget / --nothink: the think tokens {think_tokens} lie outside the "
                           f"model's vocabulary of {vocab}")


def make_parser():
    ap = argparse.ArgumentParser(prog="herbert-cli", description="Herbert - local LLM inference on MI355X")
    ap.add_argument("--arch", action="store_true", help="Show the GPU this would run on and exit")
    ap.add_argument("--model", help="Model directory")
    ap.add_argument("--backend", default="auto", help="Backend name (default: auto; use --backend help to list options)")
    ap.add_argument("--gpu", metavar="INDEX", default=None,
                    help='GPU device index. Use "list" to show available GPUs.')
    ap.add_argument("--prompt", help="Input prompt (text with a tokenizer, else comma-separated ids)")
    ap.add_argument("--prompt-file", help="Read prompt from a file")
    ap.add_argument("--system", help="System prompt (prepended with chat template)")
    ap.add_argument("--system-file", help="Read system prompt from a file")
    ap.add_argument("--max-tokens", type=int, default=2048, help="Max tokens to generate")
    ap.add_argument("--ignore-eos", action="store_true", help="Ignore EOS token")
    ap.add_argument("--no-repeat-check", action="store_true", help="Disable repetition loop detection")
    ap.add_argument("--stop", action="append", default=[],
                    help="Stop sequence (repeatable); without a tokenizer a token id")
    ap.add_argument("--verbose", action="store_true", help="Show stats after generation")
    ap.add_argument("--temperature", type=float, default=0.4, help="Sampling temperature (0 = greedy argmax)")
    ap.add_argument("--top-k", type=int, default=40, help="Top-k sampling (0 = disabled)")
    ap.add_argument("--top-p", type=float, default=0.9, help="Top-p / nucleus sampling (1.0 = disabled)")
    ap.add_argument("--think-budget", type=int, default=0,
                    help="Max tokens in <think> before forcing </think> (0 = unlimited)")
    ap.add_argument("--nothink", action="store_true", help="Disable thinking (a think block is closed at once)")
    ap.add_argument("--show-specials", action="store_true", help="Show special tokens in output")
    ap.add_argument("--prefill-chunk-size", type=int, default=None,
                    help="Process the prompt in chunks of N tokens (default: HERBERT_PREFILL_CHUNK_SIZE, else whole)")
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
    from .sampling import INTERRUPTED, SamplingParams
    if args.arch:
        return print_arch()
    # one backend here, under two names; `help` lists them, `--gpu list` the devices
    # (crates/cli/src/main.rs:367-386)
    if args.backend == "help":
        print(f"Available backends:\n  auto        the one below\n  {BACKEND}  hand-written HIP kernels for MI355X",
              file=sys.stderr)
        return 0
    if args.backend not in ("auto", BACKEND):
        raise RequestError(f"unknown backend {args.backend!r}; available: auto, {BACKEND}")
    if args.gpu == "list":
        return print_arch()
    if args.gpu is not None:
        if not args.gpu.isdigit():
            raise RequestError(f'--gpu must be a number or "list", got: {args.gpu}')
        import torch
        if int(args.gpu) >= max(1, torch.cuda.device_count()):
            raise RequestError(f"--gpu {args.gpu}: this process sees {torch.cuda.device_count()} GPU(s)")
        if torch.cuda.is_available():
            torch.cuda.set_device(int(args.gpu))
    if not args.model:
        raise RequestError("--model is required")
    if args.random_weights and not os.path.exists(os.path.join(args.model, "model.safetensors")):
        write_random_model(args.model, os.path.join(args.model, "config.json"), seed=args.seed or 0,
                           dtype=args.dtype)
    prompt = args.prompt
    if args.prompt_file:
        with open(args.prompt_file) as f:
            prompt = f.read()
    # --system wins over --system-file (crates/cli/src/main.rs:390-397)
    system = args.system
    if system is None and args.system_file:
        try:
            with open(args.system_file) as f:
                system = f.read()
        except OSError as e:
            raise RequestError(f"Failed to read system file {args.system_file!r}: {e}") from None
    # the flag, else the environment, else the prompt whole (crates/cli/src/main.rs:400-408)
    prefill_chunk = args.prefill_chunk_size
    if prefill_chunk is None:
        env = os.environ.get("HERBERT_PREFILL_CHUNK_SIZE", "")
        prefill_chunk = int(env) if env.isdigit() else None
    if prefill_chunk is not None and prefill_chunk <= 0:
        prefill_chunk = None
    tokenizer = load_tokenizer(args.model)
    from .config import load_config
    chat = load_config(args.model)[0].chat
    if prompt is None:
        if tokenizer is None or chat is None:
            raise RequestError("--prompt or --prompt-file is required: the conversation needs a tokenizer.json "
                               "and a chat template")
        from .chat import run_from_args
        return run_from_args(args, tokenizer, chat, system, prefill_chunk)
    if tokenizer is not None:
        text = chat.build_prompt(prompt, system) if chat is not None else prompt
        ids = tokenizer.encode(text, add_special_tokens=False).ids
    else:
        ids = parse_token_ids(prompt)
    stop_ids = []
    stop_strings = []
    if tokenizer is None:
        for s in args.stop:
            stop_ids.extend(parse_token_ids(s))
    else:
        stop_strings = normalize_stop_sequences(args.stop)
        end = end_of_turn_id(chat, tokenizer)
        if end is not None:
            stop_ids.append(end)

    # --nothink is a budget of one token (crates/cli/src/main.rs:685-687)
    think_budget = 1 if args.nothink else max(0, args.think_budget)
    think_tokens = think_tokens_of(chat, tokenizer) if think_budget > 0 else None

    t0 = time.perf_counter()
    cache_tokens = args.cache_tokens or (len(ids) + args.max_tokens + 65)
    engine = load(args.model, dtype=args.dtype, cache_tokens=cache_tokens)
    load_seconds = time.perf_counter() - t0

    params = SamplingParams(temperature=args.temperature, top_k=args.top_k, top_p=args.top_p,
                            max_tokens=args.max_tokens + 1, stop_ids=tuple(stop_ids),
                            ignore_eos=args.ignore_eos, repeat_check=not args.no_repeat_check,
                            seed=args.seed, think_budget=think_budget, think_tokens=think_tokens)
    check_think_tokens(think_tokens, engine.spec.vocab_size)
    on_token = StreamPrinter(tokenizer, args.show_specials, stop_strings).on_token

    interrupt = InterruptFlag().install()
    t0 = time.perf_counter()
    try:
        result = engine.generate([ids], params, on_token=on_token, interrupt=interrupt,
                                 prefill_chunk=prefill_chunk)[0]
    finally:
        interrupt.restore()
    total = time.perf_counter() - t0
    print()
    if result.stop_reason == INTERRUPTED:
        print("[herbert] Interrupted", file=sys.stderr)
    if args.verbose:
        st = engine.last_generation_stats
        decoded = max(0, st.generated_tokens - 1)
        err = sys.stderr
        print("--- Stats ---", file=err)
        print(f"Backend:         {BACKEND}", file=err)
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
