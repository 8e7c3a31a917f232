"""The conversation of the command line, in the manner of the reference's chat mode
(crates/cli/src/chat.rs:601-1331; entered where no prompt is given, crates/cli/src/main.rs:718-757).

A conversation keeps its slot of the cache: a turn's tokens go on from what earlier turns left
there (the reference's continue_prefill on a kept KvHandle, chat.rs:1060-1075), so a turn costs
its own tokens only. The commands are the reference's (chat.rs:548-572,694-806) without those of
what is not built here (tools, images, embeddings): /help /h, /quit /q /exit, /clear, /stats,
/config, /greedy, /temp, /topk, /topp, /think, /nothink, /arch, and !command for the shell; a
line that ends in a backslash goes on in the next one.

One difference in what the cache holds between two turns. The reference never puts a turn's
last generated token through the model: after a turn that the model ended itself the next
one's text follows the reply directly, and only after a turn cut short does it begin with the
end-of-turn text (chat.rs:364-381, 1046-1048). Here the next turn always begins with that last
token, then the end-of-turn token if that was not it, then what the template puts between
turns: the model sees the conversation as its template writes it.
"""
import dataclasses
import os
import subprocess
import sys
import time

from .cache import PAGE_TOKENS
from .errors import HerbertError, RequestError
from .sampling import INTERRUPTED, MAX_TOKENS, SamplingParams


class ChatSession:
    """One conversation on one engine. `say(text)` runs a turn and returns its GenerationResult;
    the totals are what /stats shows (chat.rs:713-739)."""

    def __init__(self, engine, tokenizer, chat, params, system=None, prefill_chunk=None, end_id=None):
        from .engine.generate import Generator
        self.engine, self.tokenizer, self.chat = engine, tokenizer, chat
        self.system = system
        self.params = params
        self.end_id = end_id
        self.generator = Generator(engine, max_batch=1, prefill_chunk=prefill_chunk)
        self.slot = None
        self.last_token = None          # the newest generated token: not yet through the model
        self.sampler = None
        self.turns = 0
        self.prefill_tokens = self.decode_tokens = 0
        self.prefill_seconds = self.decode_seconds = 0.0

    # ---- what the commands change
    def set_params(self, **changes):
        """Other sampling parameters from the next turn on (a new sampler: its generator stream
        starts again from the seed)."""
        params = dataclasses.replace(self.params, **changes)
        params.validate()
        self.params = params
        self.sampler = None

    def clear(self):
        """Forget the conversation: the slot goes back, the next turn is a first one (chat.rs:705-712)."""
        if self.slot is not None:
            self.engine.free_slot(self.slot)
        self.slot, self.last_token = None, None

    @property
    def held_tokens(self):
        return self.engine.cache.length(self.slot) if self.slot is not None else 0

    # ---- a turn
    def turn_tokens(self, text):
        """The tokens that a user's message adds to the sequence."""
        encode = lambda t: self.tokenizer.encode(t, add_special_tokens=False).ids
        if self.slot is None:
            return encode(self.chat.build_prompt(text, self.system))
        lead = "" if self.last_token == self.end_id else (self.chat.end_of_turn or "")
        return [self.last_token] + encode(lead + self.chat.between_turns + self.chat.build_prompt(text, None))

    def say(self, text, on_token=None, interrupt=None):
        tokens = self.turn_tokens(text)
        if not tokens:
            raise RequestError("the message produced no tokens")
        eng = self.engine
        # room: the cache's pages (all this conversation's), the model's positions; one position
        # is left for the step that may run ahead of the host
        capacity = min(eng.cache.n_pages * PAGE_TOKENS, eng.spec.max_positions)
        room = capacity - self.held_tokens - len(tokens) - 1
        if room < 1:
            raise RequestError(f"the conversation holds {self.held_tokens} tokens and this turn brings "
                               f"{len(tokens)}: no room left in {capacity} (/clear starts a new one)")
        params = self.params
        if params.max_tokens > room:
            params = dataclasses.replace(params, max_tokens=room)
        if self.sampler is None:
            from .sampling.sampler import Sampler
            self.sampler = Sampler(self.params, 1, eng.spec.vocab_size, eng.device)
        self.sampler.new_turn()
        if self.slot is None:
            self.slot = eng.alloc_slot()
        try:
            result = self.generator.extend(self.slot, tokens, params, self.sampler, on_token, interrupt)
        except BaseException:
            # (an error of the engine's, or anything the caller's on_token raised) what the slot
            # holds is no longer known to end where a turn ends: start over
            self.clear()
            raise
        st = self.generator.stats
        self.turns += 1
        self.prefill_tokens += st.prompt_tokens
        self.prefill_seconds += st.prefill_seconds
        self.decode_tokens += st.generated_tokens
        self.decode_seconds += st.decode_seconds
        self.last_token = result.tokens[-1] if result.tokens else None
        if self.last_token is None:
            self.clear()
        return result


# The commands are the reference's (crates/cli/src/chat.rs:549-572: their names and what they do,
# without those of tools, images and embeddings); the wording is this library's.
HELP = """Commands of a conversation (a line that starts with / or !):
  /help  /h        this list
  /quit  /q  /exit leave
  /clear           forget the conversation; the next message starts a new one
  /stats           turns, tokens and speeds so far
  /config          the sampling parameters in use
  /greedy          always take the most likely token (temperature 0)
  /temp <x>        temperature; 0 is greedy
  /topk <n>        keep the n most likely tokens; 0 keeps all
  /topp <p>        keep the most likely tokens up to a total probability p; 1 keeps all
  /think <n>       at most n tokens inside a <think> block; 0 lifts the limit
  /nothink         no thinking: a think block is closed as soon as it opens
  /arch            the GPU this runs on
  !<command>       run a shell command, e.g. !ls

A line that ends with \\ goes on in the next line."""


def _rate(tokens, seconds):
    return tokens / seconds if seconds > 0 else 0.0


def config_text(params, nothink):
    """What /config shows (chat.rs:574-590)."""
    lines = [f"--- Config ({'greedy' if params.greedy else 'sampling'}) ---",
             f"  temperature:  {params.temperature}", f"  top_k:        {params.top_k}",
             f"  top_p:        {params.top_p}"]
    if nothink:
        lines.append("  thinking:     disabled")
    elif params.think_budget == 0:
        lines.append("  think_budget: unlimited")
    else:
        lines.append(f"  think_budget: {params.think_budget} tokens")
    return "\n".join(lines)


class Chat:
    """The loop around a ChatSession: reads lines, runs commands and turns. `read_line(prompt)`
    returns a line or raises EOFError / KeyboardInterrupt, as `input` does; messages go to `err`
    and the model's text to `out`, as in the reference."""

    def __init__(self, session, think_tokens=None, nothink=False, show_specials=False, stop_strings=(),
                 read_line=input, out=None, err=None, make_interrupt=None):
        self.session = session
        self.think_tokens = think_tokens      # a callable that gives them (and checks them), or None
        self.nothink = nothink
        self.show_specials = show_specials
        self.stop_strings = list(stop_strings)
        self.read_line = read_line
        self.out = out if out is not None else sys.stdout
        self.err = err if err is not None else sys.stderr
        # what a turn is run under: make_interrupt() gives an object with install() (returns what the
        # generation loop asks before every step) and restore(); at the prompt signals are Python's own
        self.make_interrupt = make_interrupt

    def say(self, *lines):
        print(*lines, sep="\n", file=self.err, flush=True)

    def read_message(self):
        """One message: a line, or several joined where they end in a backslash (chat.rs:633-660).
        None at the end of the input."""
        try:
            line = self.read_line("\n>>> ")
        except EOFError:
            return None
        except KeyboardInterrupt:
            return ""
        full = ""
        while line.rstrip("\r\n").endswith("\\"):
            full += line.rstrip("\r\n")[:-1] + "\n"
            try:
                line = self.read_line("... ")
            except (EOFError, KeyboardInterrupt):
                return full
        return full + line.rstrip("\r\n")

    def _set_think(self, budget):
        changes = {"think_budget": budget}
        if budget > 0 and self.session.params.think_tokens is None:
            if self.think_tokens is None:
                self.say("This architecture names no think tokens")
                return
            changes["think_tokens"] = self.think_tokens()
        self.session.set_params(**changes)

    def command(self, line):
        """Runs a slash command; False when the conversation is to end (chat.rs:687-806,923-927)."""
        s = self.session
        cmd, _, arg = line.partition(" ")
        arg = arg.strip()

        def number(kind):
            try:
                return kind(arg)
            except ValueError:
                return None
        try:
            if cmd in ("/quit", "/q", "/exit"):
                return False
            if cmd in ("/help", "/h"):
                self.say(HELP)
            elif cmd == "/arch":
                from .cli import print_arch
                print_arch()
            elif cmd == "/clear":
                s.clear()
                self.say("[Conversation cleared]")
            elif cmd == "/stats":
                self.say("--- Chat Stats ---", f"Turns:           {s.turns}",
                         f"KV cache tokens: {s.held_tokens}" + ("" if s.slot is not None else " (cleared)"),
                         f"Prefill:         {s.prefill_tokens} tokens in {s.prefill_seconds:.3f}s "
                         f"({_rate(s.prefill_tokens, s.prefill_seconds):.1f} tok/s)",
                         f"Decode:          {s.decode_tokens} tokens in {s.decode_seconds:.3f}s "
                         f"({_rate(s.decode_tokens, s.decode_seconds):.1f} tok/s)",
                         f"Total generated: {s.decode_tokens}")
            elif cmd == "/config":
                self.say(config_text(s.params, self.nothink))
            elif cmd == "/greedy":
                s.set_params(temperature=0.0, top_k=0, top_p=1.0)
                self.say(config_text(s.params, self.nothink))
            elif cmd == "/temp":
                v = number(float)
                if v is None:
                    self.say("Usage: /temp <value>  (e.g. /temp 0.6)")
                elif v < 0:
                    self.say("Temperature must be >= 0")
                else:
                    s.set_params(temperature=v)
                    self.say(config_text(s.params, self.nothink))
            elif cmd == "/topk":
                v = number(int)
                if v is None or v < 0:
                    self.say("Usage: /topk <value>  (e.g. /topk 50)")
                else:
                    s.set_params(top_k=v)
                    self.say(config_text(s.params, self.nothink))
            elif cmd == "/topp":
                v = number(float)
                if v is None:
                    self.say("Usage: /topp <value>  (e.g. /topp 0.9)")
                elif not 0.0 <= v <= 1.0:
                    self.say("Top-p must be between 0 and 1")
                else:
                    s.set_params(top_p=v)
                    self.say(config_text(s.params, self.nothink))
            elif cmd == "/think":
                v = number(int)
                if v is None or v < 0:
                    self.say("Usage: /think <N>  (e.g. /think 200, /think 0 for unlimited)")
                else:
                    self.nothink = False
                    self._set_think(v)
                    self.say(config_text(s.params, self.nothink))
            elif cmd == "/nothink":
                # a budget of one token: a block that the model opens is closed at once (chat.rs:796-803)
                self.nothink = True
                self._set_think(1)
                self.say(config_text(s.params, self.nothink))
            elif cmd in ("/tools", "/image", "/embed", "/dist"):
                self.say(f"{cmd} is not available here (no tools, images or embedding models)")
            else:
                self.say(f"Unknown command: {cmd}. Type /help for available commands.")
        except HerbertError as e:
            self.say(f"[{e}]")
        return True

    def turn(self, text):
        from .cli import StreamPrinter
        s = self.session
        tokens = s.turn_tokens(text)
        if self.show_specials:
            # (chat.rs:1051-1058,1094-1101)
            kind = "Prompt" if s.slot is None else "Turn"
            self.say(f"--- {kind} ({len(tokens)} tokens) ---", s.tokenizer.decode(tokens, skip_special_tokens=False),
                     f"--- End {kind.lower()} ---")
        printer = StreamPrinter(s.tokenizer, self.show_specials, self.stop_strings, out=self.out)
        guard = self.make_interrupt() if self.make_interrupt is not None else None
        try:
            result = s.say(text, printer.on_token, guard.install() if guard is not None else None)
        except HerbertError as e:
            print(file=self.out, flush=True)
            self.say(f"[{e}]")
            return
        finally:
            if guard is not None:
                guard.restore()
        print(file=self.out, flush=True)
        if result.stop_reason == INTERRUPTED:
            self.say("[Interrupted]")
        elif result.stop_reason == MAX_TOKENS and len(result.tokens) < s.params.max_tokens:
            self.say("[The cache is full: /clear starts a new conversation]")

    def run(self):
        self.say("", "Type /help for commands, /quit to exit.")
        while True:
            message = self.read_message()
            if message is None:
                break
            text = message.strip()
            if not text:
                continue
            if text.startswith("!"):
                # (chat.rs:672-684)
                shell = text[1:].strip()
                if not shell:
                    self.say("Usage: !<command>  (e.g. !ls, !pwd)")
                else:
                    subprocess.run(shell, shell=True)
                continue
            if text.startswith("/"):
                if not self.command(text):
                    break
                continue
            self.turn(text)
        self.session.clear()
        return 0


def _line_reader():
    """`input` with a history in $HOME/.herbert/history.txt where that can be had (chat.rs:618-631)."""
    path = None
    try:
        import readline
        home = os.environ.get("HOME")
        if home:
            folder = os.path.join(home, ".herbert")
            os.makedirs(folder, exist_ok=True)
            path = os.path.join(folder, "history.txt")
            if os.path.exists(path):
                readline.read_history_file(path)
    except (ImportError, OSError):
        path = None

    def save():
        if path is not None:
            try:
                import readline
                readline.write_history_file(path)
            except OSError:
                pass

    def read(prompt):
        if sys.stdin.isatty():
            return input(prompt)
        line = sys.stdin.readline()       # lines from a pipe: no prompt among the model's text
        if not line:
            raise EOFError
        return line
    return read, save


def run_from_args(args, tokenizer, chat, system, prefill_chunk):
    """The command line's chat mode: the options mean what they mean for a single prompt,
    --max-tokens counting a turn's tokens as the reference's chat counts them
    (`for _ in 1..max_tokens` after the first, chat.rs:231)."""
    from .api import load
    from .cli import (InterruptFlag, check_think_tokens, end_of_turn_id, normalize_stop_sequences,
                      think_tokens_of)
    end = end_of_turn_id(chat, tokenizer)
    think_budget = 1 if args.nothink else max(0, args.think_budget)
    think_tokens = think_tokens_of(chat, tokenizer) if think_budget > 0 else None
    t0 = time.perf_counter()
    engine = load(args.model, dtype=args.dtype, cache_tokens=args.cache_tokens or 16384)
    if args.verbose:
        print(f"Model load:      {time.perf_counter() - t0:.3f}s", file=sys.stderr)
    check_think_tokens(think_tokens, engine.spec.vocab_size)

    def later_think_tokens():
        found = think_tokens_of(chat, tokenizer)
        check_think_tokens(found, engine.spec.vocab_size)
        return found

    params = SamplingParams(temperature=args.temperature, top_k=args.top_k, top_p=args.top_p,
                            max_tokens=max(1, args.max_tokens), stop_ids=(end,) if end is not None else (),
                            ignore_eos=False, repeat_check=not args.no_repeat_check, seed=args.seed,
                            think_budget=think_budget, think_tokens=think_tokens)
    session = ChatSession(engine, tokenizer, chat, params, system=system, prefill_chunk=prefill_chunk, end_id=end)
    read_line, save_history = _line_reader()
    try:
        return Chat(session, think_tokens=later_think_tokens, nothink=args.nothink, show_specials=args.show_specials,
                    stop_strings=normalize_stop_sequences(args.stop), read_line=read_line,
                    make_interrupt=InterruptFlag).run()
    finally:
        save_history()
