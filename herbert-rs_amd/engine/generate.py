"""The generation loop above the step function.

Requests are served in batches, one after another: the prompts of a batch in
one step, then one token for every sequence that still runs. A sequence ends
on its end-of-sequence token (kept in the output, as the reference keeps it:
crates/cli/src/main.rs:1272,1357-1359), on a stop token, after max_tokens
tokens, on a repetition loop (crates/core/src/decode_utils.rs:14-33), when
the caller's `on_token` says so (stop strings are the caller's, since text is:
crates/cli/src/main.rs:1328-1332,1360) or at the model's last position; it
gives its slot back at once and the others go on. Before every decode step
the caller's interrupt flag is looked at (crates/cli/src/main.rs:1242-1245):
when it is set, every running sequence ends with what it has and every slot
is given back.

Where engine and sampler allow it, decode steps are put on the GPU's stream
one ahead of the host (`_decode_ahead`): a step takes its tokens from where
the sampler left them on the GPU, and the host reads them, applies the stop
rules and calls `on_token` while the next step already runs. The tokens and
stop reasons are those of the step-by-step loop.

`max_tokens` here counts every generated token, the one the prompt's step
gives included: the reference's chat and server loops (`for _ in
1..max_tokens` after the first token, crates/cli/src/chat.rs:231). Its
single-shot command line runs `for _step in 0..max_tokens` decode steps after
the first token (crates/cli/src/main.rs:1040,1241), one token more; the
command line here asks this loop for max_tokens + 1 to give what that gives.
"""
import time
from dataclasses import dataclass, field
from typing import List

from ..cache import PAGE_TOKENS
from ..errors import BackendError, RequestError
from ..sampling import (EOS, INTERRUPTED, LENGTH, MAX_TOKENS, REPETITION_LOOP, STOP_TOKEN,
                        SamplingParams, detect_repetition_loop)
from .batch import StepEntry


@dataclass
class GenerationResult:
    tokens: List[int]
    stop_reason: str
    prompt_tokens: int


@dataclass
class GenerationStats:
    prompt_tokens: int = 0
    generated_tokens: int = 0
    prefill_seconds: float = 0.0
    decode_seconds: float = 0.0
    decode_steps: int = 0
    batches: int = 0


def _rounded(n):
    return (n + PAGE_TOKENS - 1) // PAGE_TOKENS * PAGE_TOKENS


def plan_batches(prompt_lengths, max_new, max_batch, capacity_tokens, max_positions):
    """Lists of request indices, in order, each list one batch that fits the cache."""
    batches, current, used = [], [], 0
    for i, n in enumerate(prompt_lengths):
        if n <= 0:
            raise RequestError(f"request {i} has an empty prompt")
        if n > max_positions:
            raise RequestError(f"request {i}: prompt of {n} tokens exceeds "
                               f"max_position_embeddings ({max_positions})")
        need = _rounded(min(n + max_new, max_positions))
        if need > capacity_tokens:
            raise RequestError(f"request {i} needs room for {need} tokens but the cache holds "
                               f"{capacity_tokens}")
        if current and (len(current) >= max_batch or used + need > capacity_tokens):
            batches.append(current)
            current, used = [], 0
        current.append(i)
        used += need
    if current:
        batches.append(current)
    return batches


def stop_reason(generated, params, eos_id):
    """Why a sequence ends after its newest token, or None."""
    tok = generated[-1]
    if not params.ignore_eos and eos_id is not None and tok == eos_id:
        return EOS
    if tok in params.stop_ids:
        return STOP_TOKEN
    if len(generated) >= params.max_tokens:
        return MAX_TOKENS
    if params.repeat_check and detect_repetition_loop(generated) is not None:
        return REPETITION_LOOP
    return None


class Generator:
    """Runs requests through an engine. `make_chooser(params, n, vocab, device)` builds the object
    whose `choose(logits, sequence_indices)` picks tokens (the GPU sampler by default)."""

    def __init__(self, engine, max_batch=64, make_chooser=None, prefill_chunk=None, run_ahead=True):
        self.engine = engine
        self.max_batch = int(max_batch)
        # decode steps are put on the GPU's stream one ahead of the host where engine and chooser can
        self.run_ahead = bool(run_ahead)
        # prompts longer than this many tokens are fed in pieces of that size, one step a piece
        # (the reference's prefill_chunk_size: crates/cli/src/main.rs:400-408)
        self.prefill_chunk = int(prefill_chunk) if prefill_chunk else None
        if self.prefill_chunk is not None and self.prefill_chunk <= 0:
            raise RequestError("prefill_chunk must be > 0")
        if make_chooser is None:
            from ..sampling.sampler import Sampler
            make_chooser = Sampler
        self.make_chooser = make_chooser
        self.stats = GenerationStats()
        # the loop is done with a decode step's logits before its next step: it takes the engine's
        # own rows where the engine would otherwise hand out a copy
        self._views = {"keep_logits": False} if getattr(engine, "hands_out_copies", False) else {}

    def generate(self, prompts, params=None, on_token=None, interrupt=None):
        """One GenerationResult per prompt (a list of token ids), in the prompts' order.
        on_token(request index, token) is called for every generated token; if it returns a
        string, the sequence ends there with that stop reason (the token is kept). It must not
        use the engine: the step after the token's may already be on the GPU. `interrupt()`
        is asked before every decode step and before every batch: once it is true, running
        sequences end with reason "interrupted" and requests not yet started return no tokens."""
        params = params or SamplingParams()
        params.validate()
        eng = self.engine
        spec = eng.spec
        capacity = eng.cache.n_pages * PAGE_TOKENS
        batches = plan_batches([len(p) for p in prompts], params.max_tokens, self.max_batch,
                               capacity, spec.max_positions)
        chooser = self.make_chooser(params, len(prompts), spec.vocab_size, eng.device)
        results = [None] * len(prompts)
        self.stats = GenerationStats()
        for members in batches:
            if interrupt is not None and interrupt():
                for i in members:
                    results[i] = GenerationResult([], INTERRUPTED, len(prompts[i]))
                continue
            self._run_batch(members, prompts, params, chooser, results, on_token, interrupt)
            self.stats.batches += 1
        return results

    def _prompts(self, live, prompts, slots, chooser):
        """The prompts of a batch through the engine; the first token of each sequence, in the
        order of `live`. Whole in one step, or, with a prefill chunk, in steps that carry the
        next piece of every prompt that still has one: a sequence's token is chosen in the step
        that brings its last piece."""
        eng, chunk = self.engine, self.prefill_chunk
        if chunk is None or all(len(prompts[i]) <= chunk for i in live):
            entries = [StepEntry(slots[i], list(prompts[i]), [len(prompts[i]) - 1]) for i in live]
            return chooser.choose(eng.step(entries), list(live))
        fed = {i: 0 for i in live}
        first = {}
        while len(first) < len(live):
            entries, ending = [], []
            for i in live:
                left = len(prompts[i]) - fed[i]
                if left <= 0:
                    continue
                n = min(chunk, left)
                entries.append(StepEntry(slots[i], list(prompts[i][fed[i]:fed[i] + n]), [n - 1] if n == left else []))
                if n == left:
                    ending.append(i)
                fed[i] += n
            logits = eng.step(entries)
            if ending:
                first.update(zip(ending, chooser.choose(logits, ending)))
        return [first[i] for i in live]

    def _decode_ahead(self, live, slots, generated, params, chooser, take, kept=()):
        """Decoding with the host one step behind the GPU. The tokens that a step chooses stay on
        the GPU, and the next step is put on the stream with them at once, before the host has
        seen them; the host reads a step's tokens while the next one runs, so the GPU does not
        wait for the host's share of a step. A sequence whose newest token turns out to end it
        (end of sequence, a stop token, the caller's word) has then already been through one step
        more: that step's work on it is thrown away, its slot is given back as always, and every
        other sequence's tokens are what they would have been. Sequences that end for a reason the
        host knows beforehand (max_tokens, the model's last position) are not taken ahead.
        The step thrown away has also taken a draw from the sequence's generator stream: for a
        sequence whose slot the caller keeps (`kept`: its chooser goes on into the next turn) the
        streams are saved before every step that runs ahead (`chooser.save_streams`) and the
        sequence's is put back when it ends, so that a seeded conversation draws what the
        step-by-step loop draws, one draw a token."""
        eng = self.engine
        saves = bool(kept) and hasattr(chooser, "save_streams")

        def launch(order, device_tokens):
            entries = [StepEntry(slots[i], [generated[i][-1]] if device_tokens is None else [0], [0])
                       for i in order]
            logits = eng.step(entries, tokens_on_device=device_tokens, **self._views)
            self.stats.decode_steps += 1
            return chooser.choose_ahead(logits, order), {i: eng.cache.length(slots[i]) for i in order}

        if not live:
            return
        order = list(live)
        pending, held = launch(order, None)
        while True:
            # the step after the one in flight, for the sequences that its token cannot end by count
            ahead = [i for i in order if i in slots and len(generated[i]) + 2 <= params.max_tokens
                     and eng.cache.length(slots[i]) < eng.spec.max_positions]
            following = saved = None
            if ahead:
                rows = [order.index(i) for i in ahead]
                if saves:
                    saved = chooser.save_streams()
                following = launch(ahead, chooser.rows_of(pending, rows))
            take(order, chooser.read(pending), held)
            if saved is not None:
                for i in ahead:
                    if i not in slots and i in kept:        # it ended on this token: the draw after it never was
                        chooser.restore_stream(i, saved)
            if not live or following is None:
                break
            order, (pending, held) = ahead, following

    def extend(self, slot, tokens, params, chooser, on_token=None, interrupt=None):
        """One more turn of a sequence whose slot the caller keeps (the reference's
        continue_prefill and decode on a kept KvHandle, crates/cli/src/chat.rs:1060-1075,
        164-352): `tokens` go on from what the slot holds (nothing, for a first turn), then
        tokens are generated as in `generate`. The slot is not given back; when this returns it
        holds everything up to the newest generated token, which itself has not been through
        the model: the next turn's tokens begin with it. `chooser` is the caller's too (its
        generator streams go on from turn to turn); sequence index 0 is used. Returns one
        GenerationResult."""
        params.validate()
        if not tokens:
            raise RequestError("a turn needs at least one token")
        eng = self.engine
        room = eng.spec.max_positions - eng.cache.length(slot)
        if len(tokens) > room:
            raise RequestError(f"a turn of {len(tokens)} tokens does not fit: the sequence holds "
                               f"{eng.cache.length(slot)} of max_position_embeddings ({eng.spec.max_positions})")
        results = [None]
        self.stats = GenerationStats()
        self._run_batch([0], [list(tokens)], params, chooser, results, on_token, interrupt, kept={0: slot})
        self.stats.batches += 1
        return results[0]

    def _run_batch(self, members, prompts, params, chooser, results, on_token, interrupt=None, kept=None):
        """`kept`: request index -> a slot of the caller's (see `extend`) instead of one taken
        here and given back at the end."""
        eng = self.engine
        eos = eng.spec.eos_token_id
        kept = kept or {}
        slots = {i: kept[i] if i in kept else eng.alloc_slot() for i in members}
        before = {i: eng.cache.length(kept[i]) for i in kept}
        generated = {i: [] for i in members}
        live = list(members)

        def finish(i, reason):
            results[i] = GenerationResult(generated[i], reason, len(prompts[i]))
            slot = slots.pop(i)
            if i in kept:
                # a step that ran ahead of the host has taken the newest token in already
                eng.truncate(slot, before[i] + len(prompts[i]) + len(generated[i]) - 1)
            else:
                eng.free_slot(slot)
            live.remove(i)

        try:
            t0 = time.perf_counter()
            tokens = self._prompts(live, prompts, slots, chooser)
            self.stats.prefill_seconds += time.perf_counter() - t0
            self.stats.prompt_tokens += sum(len(prompts[i]) for i in live)
            t0 = time.perf_counter()

            def take(order, tokens, held=None):
                """The newest tokens of the sequences `order` (those that have ended since are
                skipped). `held`: the positions each sequence held when the step that chose these
                tokens had been put on the stream, if a later step has been since."""
                for i, tok in zip(order, tokens):
                    if i not in slots:
                        continue
                    if not 0 <= int(tok) < eng.spec.vocab_size:
                        # (the chooser's answer for a row of logits without a finite value: what a
                        # token id out of range, fed from the GPU where no host check sees it, leaves)
                        raise BackendError(f"request {i}: no token could be chosen (got {int(tok)}): its logits "
                                           "hold no finite value")
                    generated[i].append(int(tok))
                    self.stats.generated_tokens += 1
                    said = on_token(i, int(tok)) if on_token is not None else None
                    reason = stop_reason(generated[i], params, eos)
                    if reason is None and isinstance(said, str):
                        reason = said
                    length = eng.cache.length(slots[i]) if held is None else held[i]
                    if reason is None and length >= eng.spec.max_positions:
                        reason = LENGTH
                    if reason is not None:
                        finish(i, reason)
                if live and interrupt is not None and interrupt():
                    for i in list(live):
                        finish(i, INTERRUPTED)

            take(list(live), tokens)
            # (a kept slot is rolled back by the one step that ran ahead: only where the cache can)
            if self.run_ahead and getattr(chooser, "can_run_ahead", False) and \
                    getattr(eng, "accepts_device_tokens", False) and \
                    (not kept or getattr(eng.cache, "rolls_back_freely", False)):
                self._decode_ahead(live, slots, generated, params, chooser, take, kept)
            else:
                while live:
                    order = list(live)
                    logits = eng.step([StepEntry(slots[i], [generated[i][-1]], [0]) for i in order], **self._views)
                    self.stats.decode_steps += 1
                    take(order, chooser.choose(logits, order))
            self.stats.decode_seconds += time.perf_counter() - t0
        finally:
            for i in list(slots):
                slot = slots.pop(i)
                if i not in kept:
                    eng.free_slot(slot)
