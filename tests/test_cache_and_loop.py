"""The cache's bookkeeping (no slot or page lost, held twice or freed twice) and the generation
loop's decisions, on the CPU with a stand-in for the engine's step."""
import random

import numpy as np
import pytest
import torch

from herbert_rs_amd.cache import Cache, FreeList, KVNeed, StateNeed, pages_for
from herbert_rs_amd.engine.generate import Generator, plan_batches, stop_reason
from herbert_rs_amd.errors import CacheError, RequestError
from herbert_rs_amd.sampling import (EOS, INTERRUPTED, LENGTH, MAX_TOKENS, REPETITION_LOOP,
                                     STOP_SEQUENCE, STOP_TOKEN, SamplingParams, detect_repetition_loop)
from herbert_rs_amd.sampling import xorshift


def test_free_list_is_strict():
    fl = FreeList(3, "slot")
    a, b, c = fl.take(), fl.take(), fl.take()
    assert sorted((a, b, c)) == [0, 1, 2]
    with pytest.raises(CacheError, match="no free slot"):
        fl.take()
    fl.give_back(b)
    with pytest.raises(CacheError, match="freed twice"):
        fl.give_back(b)
    with pytest.raises(CacheError):
        fl.give_back(7)
    assert fl.take() == b
    fl.check()


def make_cache(window=None, state=False, max_tokens=64 * 12, max_positions=512):
    needs = {0: KVNeed(2, 8, None), 1: KVNeed(2, 8, window), 2: KVNeed(2, 8, None)}
    if state:
        needs[3] = StateNeed((4,), torch.float32)
        needs[1] = (KVNeed(2, 8, window), StateNeed((4,), torch.float32))
    return Cache(needs, max_tokens, max_positions, torch.float32, "cpu")


def test_groups_have_storage_of_their_own():
    c = make_cache(window=100)
    assert len(c.kv_groups) == 2
    full = c.kv_groups[KVNeed(2, 8, None)]
    win = c.kv_groups[KVNeed(2, 8, 100)]
    assert full.entries == [0, 2] and win.entries == [1]
    # twelve pages for sequences and the padding page, which only the padding slot's table names
    assert full.pool.shape == (2, 2, 13, 2, 64, 8) and win.pool.shape == (1, 2, 13, 2, 64, 8)
    assert c.pad_slot == c.n_slots == 12 and full.pages.count == 12
    assert full.table.shape[0] == 13 and set(full.table[c.pad_slot].tolist()) == {12}
    assert 12 not in set(full.table[:12].flatten().tolist())
    assert c.kv_view(0).k.data_ptr() != c.kv_view(2).k.data_ptr()
    assert c.kv_view(1).window == 100 and c.kv_view(0).window == 0


def test_pages_follow_lengths_and_come_back():
    c = make_cache()
    s = c.alloc_slot()
    g = c.kv_groups[KVNeed(2, 8, None)]
    c.reserve(s, 5); c.commit(s, 5)
    assert g.pages.held_count == 1
    c.reserve(s, 59); c.commit(s, 59)
    assert g.pages.held_count == 1 and c.length(s) == 64
    c.reserve(s, 1); c.commit(s, 1)
    assert g.pages.held_count == 2
    assert g.table[s, :2].tolist() == g.table_host[s, :2].tolist()
    c.check()
    c.free_slot(s)
    assert g.pages.held_count == 0
    c.check()
    with pytest.raises(CacheError):
        c.free_slot(s)
    with pytest.raises(CacheError):
        c.length(s)


def test_window_group_gives_back_unseen_pages():
    c = make_cache(window=70)
    s = c.alloc_slot()
    win = c.kv_groups[KVNeed(2, 8, 70)]
    full = c.kv_groups[KVNeed(2, 8, None)]
    c.reserve(s, 200); c.commit(s, 200)
    # the next query (position 200) sees keys 131..200: pages 0 and 1 (keys 0..127) are out of sight
    assert win.first_page[s] == 2 and win.pages.held_count == 2 and full.pages.held_count == 4
    for _ in range(60):
        c.reserve(s, 1); c.commit(s, 1)
    assert win.first_page[s] == 2 + (261 - 70 - 128) // 64 and c.length(s) == 260
    c.check()
    with pytest.raises(CacheError, match="given up"):
        c.truncate(s, 100)
    c.truncate(s, 250)
    assert c.length(s) == 250
    c.free_slot(s)
    assert win.pages.held_count == 0 and full.pages.held_count == 0
    c.check()


def test_exhaustion_and_limits():
    c = make_cache(max_tokens=64 * 3)
    a, b = c.alloc_slot(), c.alloc_slot()
    c.reserve(a, 128); c.commit(a, 128)
    with pytest.raises(CacheError, match="no free page"):
        c.reserve(b, 129)
    c.free_slot(b)
    c.free_slot(a)
    c.check()
    s = c.alloc_slot()
    with pytest.raises(CacheError, match="exceed"):
        c.reserve(s, 513)
    assert Cache({0: KVNeed(1, 8)}, 100, 512, torch.float32, "cpu").n_pages == 2    # rounded up to 64


def test_state_is_cleared_when_a_slot_is_taken_again():
    c = make_cache(state=True)
    s = c.alloc_slot()
    views = c.state_views(1)
    assert len(views) == 1 and views[0].shape == (c.n_slots + 1, 4)          # the last row: the padding slot
    views[0][s] = 5.0
    c.state_views(3)[0][s] = 2.0
    c.free_slot(s)
    s2 = c.alloc_slot()
    assert s2 == s
    assert float(c.state_views(1)[0][s2].abs().sum()) == 0 and float(c.state_views(3)[0][s2].abs().sum()) == 0
    c.reserve(s2, 3); c.commit(s2, 3)
    with pytest.raises(CacheError, match="rolled back"):
        c.truncate(s2, 1)


def test_random_walk_keeps_the_books():
    rnd = random.Random(3)
    c = make_cache(window=70, max_tokens=64 * 40)
    live = {}
    for _ in range(400):
        r = rnd.random()
        if r < 0.3 and len(live) < 10:
            live[c.alloc_slot()] = 0
        elif r < 0.5 and live:
            s = rnd.choice(list(live))
            c.free_slot(s)
            del live[s]
        elif live:
            s = rnd.choice(list(live))
            n = rnd.choice([1, 1, 1, 7, 64, 90])
            if live[s] + n <= 512:
                try:
                    c.reserve(s, n)
                except CacheError:
                    continue
                c.commit(s, n)
                live[s] += n
        c.check()
        for s, n in live.items():
            assert c.length(s) == n
            full = c.kv_groups[KVNeed(2, 8, None)].table_host[s]
            assert (full >= 0).sum() == pages_for(n)
    for s in list(live):
        c.free_slot(s)
    c.check()
    assert all(g.pages.held_count == 0 for g in c.kv_groups.values())


# ---- the generation loop with a stand-in engine
class FakeCache:
    def __init__(self, n_pages):
        self.n_pages = n_pages
        self.slots = FreeList(64, "slot")
        self.lengths = {}

    def length(self, slot):
        return self.lengths[slot]


class FakeSpec:
    vocab_size = 50
    max_positions = 40
    eos_token_id = 9


class FakeEngine:
    """Logits that make the next token (last token + 1) mod vocab: the loop's decisions show."""
    device = "cpu"

    def __init__(self, n_pages=64):
        self.spec = FakeSpec()
        self.cache = FakeCache(n_pages)
        self.steps = []
        self.max_held = 0

    def alloc_slot(self):
        s = self.cache.slots.take()
        self.cache.lengths[s] = 0
        self.max_held = max(self.max_held, self.cache.slots.held_count)
        return s

    def free_slot(self, s):
        self.cache.slots.give_back(s)
        del self.cache.lengths[s]

    def step(self, entries):
        self.steps.append([(e.slot, len(e.tokens)) for e in entries])
        rows = []
        for e in entries:
            self.cache.lengths[e.slot] += len(e.tokens)
            for j in e.want:
                row = np.zeros(self.spec.vocab_size, dtype=np.float32)
                row[(e.tokens[j] + 1) % self.spec.vocab_size] = 1.0
                rows.append(row)
        return np.stack(rows) if rows else None


class ArgmaxChooser:
    def __init__(self, params, n, vocab, device):
        self.calls = []

    def choose(self, logits, sequence_indices):
        self.calls.append(list(sequence_indices))
        return [int(r.argmax()) for r in logits]


def run(prompts, engine=None, on_token=None, interrupt=None, **kw):
    engine = engine or FakeEngine()
    gen = Generator(engine, max_batch=kw.pop("max_batch", 4), make_chooser=ArgmaxChooser)
    params = SamplingParams(temperature=0.0, **kw)
    return engine, gen, gen.generate(prompts, params, on_token, interrupt)


def test_stops_eos_max_tokens_stop_token_and_order():
    eng, gen, res = run([[5], [20, 21], [7, 8]], max_tokens=6, stop_ids=(23,), repeat_check=False)
    assert res[0].tokens == [6, 7, 8, 9] and res[0].stop_reason == EOS         # eos kept in the output
    assert res[1].tokens == [22, 23] and res[1].stop_reason == STOP_TOKEN
    assert res[2].tokens == [9] and res[2].stop_reason == EOS                  # the prompt's own token
    assert [r.prompt_tokens for r in res] == [1, 2, 2]
    # one prompt step with all three, then only the unfinished ones, one token each
    assert eng.steps[0] == [(0, 1), (1, 2), (2, 2)]
    assert eng.steps[1] == [(0, 1), (1, 1)] and eng.steps[2:] == [[(0, 1)], [(0, 1)]]
    assert eng.cache.slots.held_count == 0
    assert gen.stats.generated_tokens == 7 and gen.stats.decode_steps == 3 and gen.stats.prompt_tokens == 5


def test_the_interrupt_flag_is_looked_at_before_every_decode_step():
    """crates/cli/src/main.rs:1242-1245: the flag ends the loop between two steps; what was
    generated stays, every slot comes back, batches not yet started do not start."""
    asked = []

    def interrupt():
        asked.append(1)
        return len(asked) > 3        # true when asked the fourth time

    eng, gen, res = run([[10], [20], [30]], max_tokens=20, max_batch=2, repeat_check=False,
                        interrupt=interrupt)
    # asked before the batch, then before decode steps 1, 2 and 3: two decode steps ran
    assert res[0].tokens == [11, 12, 13] and res[1].tokens == [21, 22, 23]
    assert res[0].stop_reason == res[1].stop_reason == INTERRUPTED
    assert res[2].tokens == [] and res[2].stop_reason == INTERRUPTED
    assert len(eng.steps) == 3 and eng.cache.slots.held_count == 0
    # set during the prompt's step: the token of that step is kept; a sequence that has ended
    # by itself keeps its own reason
    calls = []
    _, _, res = run([[7], [8]], max_tokens=20, repeat_check=False,
                    interrupt=lambda: calls.append(1) or len(calls) > 1)
    assert res[0].stop_reason == INTERRUPTED and res[0].tokens == [8]
    assert res[1].stop_reason == EOS and res[1].tokens == [9]


def test_the_caller_ends_a_sequence_from_on_token():
    """Stop strings are matched by whoever has the text (crates/cli/src/main.rs:1328-1332,1360):
    on_token's answer ends that sequence, the token stays in the output, the others go on."""
    def on_token(i, tok):
        return STOP_SEQUENCE if (i == 1 and tok == 23) else None
    eng, _, res = run([[10], [20]], max_tokens=5, repeat_check=False, on_token=on_token)
    assert res[1].tokens == [21, 22, 23] and res[1].stop_reason == STOP_SEQUENCE
    assert res[0].tokens == [11, 12, 13, 14, 15] and res[0].stop_reason == MAX_TOKENS
    assert eng.steps[3] == [(0, 1)] and eng.cache.slots.held_count == 0
    # the loop's own rules come first: eos on the same token is eos
    _, _, res = run([[7]], max_tokens=5, repeat_check=False, on_token=lambda i, t: STOP_SEQUENCE)
    assert res[0].tokens == [8] and res[0].stop_reason == STOP_SEQUENCE
    _, _, res = run([[8]], max_tokens=5, repeat_check=False, on_token=lambda i, t: STOP_SEQUENCE)
    assert res[0].tokens == [9] and res[0].stop_reason == EOS


def test_a_step_that_does_not_fit_takes_no_page():
    """All the pages of a step or none: the third sequence's pages do not fit, and the first
    two hold afterwards exactly what they held before."""
    c = make_cache(max_tokens=64 * 4)
    a, b, d = c.alloc_slot(), c.alloc_slot(), c.alloc_slot()
    c.reserve_all([(a, 60), (b, 10)])
    c.commit(a, 60); c.commit(b, 10)
    before = {k: (g.pages.held_count, g.table_host.copy()) for k, g in c.kv_groups.items()}
    with pytest.raises(CacheError, match="needs 4 more pages"):
        c.reserve_all([(a, 10), (b, 60), (d, 70)])       # 1 + 1 + 2 pages, 2 free
    for k, g in c.kv_groups.items():
        assert g.pages.held_count == before[k][0] and (g.table_host == before[k][1]).all()
    c.check()
    with pytest.raises(CacheError, match="exceed"):
        c.reserve_all([(a, 1), (b, 600)])
    c.reserve_all([(a, 10), (b, 60)])                    # this fits: 2 pages
    assert all(g.pages.free_count == 0 for g in c.kv_groups.values())
    c.unreserve(a); c.unreserve(b)                       # the step did not run
    for k, g in c.kv_groups.items():
        assert g.pages.held_count == before[k][0] and (g.table_host == before[k][1]).all()
    assert c.length(a) == 60 and c.length(b) == 10
    c.check()


def test_max_tokens_counts_the_first_token_and_ignore_eos():
    """The loop's max_tokens is the number of tokens that come out, the prompt step's token
    included (crates/cli/src/chat.rs:231 `for _ in 1..max_tokens` after the first token). The
    single-shot command line counts decode steps after that token
    (crates/cli/src/main.rs:1040,1241) and therefore asks the loop for one more."""
    _, _, res = run([[5]], max_tokens=3, repeat_check=False)
    assert res[0].tokens == [6, 7, 8] and res[0].stop_reason == MAX_TOKENS
    _, _, res = run([[7]], max_tokens=4, ignore_eos=True, repeat_check=False)
    assert res[0].tokens == [8, 9, 10, 11] and res[0].stop_reason == MAX_TOKENS


def test_batches_follow_one_another_and_slots_are_used_again():
    prompts = [[i] for i in (10, 11, 12, 13, 14, 15, 30)]
    eng, gen, res = run(prompts, max_tokens=2, max_batch=3, repeat_check=False)
    assert [r.tokens for r in res] == [[p[0] + 1, p[0] + 2] for p in prompts]
    assert gen.stats.batches == 3 and eng.max_held == 3
    firsts = [s for s in eng.steps if all(n == 1 for _, n in s)][::2]
    assert [sorted(slot for slot, _ in s) for s in firsts] == [[0, 1, 2], [0, 1, 2], [0]]


def test_the_model_s_last_position_ends_a_sequence():
    eng, _, res = run([list(range(10, 48))], max_tokens=10, repeat_check=False)     # 38 of 40 positions
    assert res[0].stop_reason == LENGTH and len(res[0].tokens) == 3
    assert eng.cache.slots.held_count == 0


def test_plan_batches_respects_capacity():
    assert plan_batches([5, 11, 2, 300], 8, 3, 1024, 512) == [[0, 1, 2], [3]]
    assert plan_batches([100, 100, 100], 28, 8, 256, 512) == [[0, 1], [2]]
    with pytest.raises(RequestError, match="empty"):
        plan_batches([3, 0], 8, 4, 1024, 512)
    with pytest.raises(RequestError, match="exceeds"):
        plan_batches([600], 8, 4, 4096, 512)
    with pytest.raises(RequestError, match="holds"):
        plan_batches([100], 100, 4, 128, 512)


def test_stop_reason_rules():
    p = SamplingParams(temperature=0.0, max_tokens=100, stop_ids=(4,))
    assert stop_reason([1, 2, 9], p, 9) == EOS
    assert stop_reason([1, 2, 4], p, 9) == STOP_TOKEN
    assert stop_reason([1, 2, 3], p, 9) is None
    loop = [1, 2, 3, 5, 6, 7] * 3
    assert stop_reason(loop, p, 9) == REPETITION_LOOP
    assert stop_reason(loop, SamplingParams(temperature=0.0, max_tokens=100, repeat_check=False), 9) is None
    assert stop_reason([1] * 5, SamplingParams(temperature=0.0, max_tokens=5, repeat_check=False), 9) == MAX_TOKENS
    assert detect_repetition_loop([1, 2, 3, 4, 5] * 3) is None


def test_slots_come_back_when_a_step_fails():
    class Failing(FakeEngine):
        def step(self, entries):
            if len(self.steps) == 1:
                raise RuntimeError("boom")
            return super().step(entries)
    eng = Failing()
    with pytest.raises(RuntimeError):
        run([[1], [2]], engine=eng, max_tokens=5, repeat_check=False)
    assert eng.cache.slots.held_count == 0


def test_params_are_checked_and_seeds_give_streams():
    with pytest.raises(RequestError):
        SamplingParams(temperature=-1.0).validate()
    with pytest.raises(RequestError):
        SamplingParams(max_tokens=0).validate()
    d = SamplingParams()
    assert (d.temperature, d.top_k, d.top_p, d.max_tokens) == (0.4, 40, 0.9, 2048)   # the reference's defaults
    assert xorshift.initial_state(0) == 0xDEADBEEF and xorshift.step(1) == 1082269761
    assert xorshift.sequence_seed(7, 0) == 7
    assert len({xorshift.sequence_seed(7, i) for i in range(16)}) == 16


def test_prompts_in_pieces_give_the_same_tokens():
    """With a prefill chunk the prompts go through the engine in steps that carry the next piece
    of every prompt that still has one; a sequence's first token is chosen in the step of its
    last piece, and decoding goes on as without pieces."""
    prompts = [[1, 2, 3, 4, 5], [20, 21], [30, 31, 32, 33, 34, 35, 36, 37, 38]]
    _, _, whole = run(prompts, max_tokens=3, repeat_check=False)
    eng = FakeEngine()
    gen = Generator(eng, max_batch=4, make_chooser=ArgmaxChooser, prefill_chunk=4)
    res = gen.generate(prompts, SamplingParams(temperature=0.0, max_tokens=3, repeat_check=False))
    assert [r.tokens for r in res] == [r.tokens for r in whole]
    assert eng.steps[:3] == [[(0, 4), (1, 2), (2, 4)], [(0, 1), (2, 4)], [(2, 1)]]
    assert eng.steps[3] == [(0, 1), (1, 1), (2, 1)]                  # then one token each
    assert gen.stats.prompt_tokens == 16 and eng.cache.slots.held_count == 0
    # prompts no longer than the chunk: one step as before
    eng2 = FakeEngine()
    Generator(eng2, make_chooser=ArgmaxChooser, prefill_chunk=16).generate(
        prompts, SamplingParams(temperature=0.0, max_tokens=1))
    assert eng2.steps == [[(0, 5), (1, 2), (2, 9)]]
    with pytest.raises(RequestError):
        Generator(FakeEngine(), prefill_chunk=-1)


def test_think_budget_follows_the_plain_rule():
    from herbert_rs_amd.sampling import ThinkBudget, ThinkTokens
    from .plain.sampler import think_forced
    ids = ThinkTokens(open_id=5, close_id=6, newline_id=7)
    # by hand: budget 3: after <think> a b the line break is forced, then </think>, then nothing
    tb, seen = ThinkBudget(3, ids), []
    for tok in (1, 5, 2, 2, 7, 6, 2):
        seen.append(tb.forced())
        tb.track(tok)
    assert seen == [None, None, None, None, 7, 6, None]
    # a budget of one (the command line's --nothink): line break, then the closing token
    tb, seen = ThinkBudget(1, ids), []
    for tok in (5, 7, 6, 3):
        seen.append(tb.forced())
        tb.track(tok)
    assert seen == [None, 7, 6, None]
    # a model that ignores nothing is forced nothing; a block opened by the prompt counts from there
    tb = ThinkBudget(2, ids)
    tb.set_in_think()
    assert tb.forced() is None
    tb.track(9)
    assert tb.forced() == 7
    # random streams, every prefix, against the rule written over the whole history
    rng = np.random.default_rng(3)
    for budget in (0, 1, 2, 5):
        for _ in range(40):
            stream = rng.choice([1, 2, 3, 5, 6, 7], size=30, p=[0.25, 0.25, 0.2, 0.12, 0.08, 0.1]).tolist()
            tb, history = ThinkBudget(budget, ids), []
            for tok in stream:
                want = think_forced(history, budget, 5, 6, 7)
                assert tb.forced() == want, (budget, history)
                tok = want if want is not None else tok
                tb.track(tok)
                history.append(tok)
    with pytest.raises(RequestError, match="think_tokens"):
        SamplingParams(think_budget=3).validate()


class AheadEngine(FakeEngine):
    """A stand-in engine that takes a step's tokens from "the device" (here: an array)."""
    accepts_device_tokens = True

    def step(self, entries, tokens_on_device=None):
        if any(len(e.tokens) > 1 or e.want != [0] for e in entries) or self.cache.lengths[entries[0].slot] == 0:
            AheadChooser.unread = 0          # a new batch: what ran ahead for nothing before it is forgotten
        if tokens_on_device is not None:
            assert len(tokens_on_device) == len(entries) and all(e.tokens == [0] for e in entries)
            entries = [type(e)(e.slot, [int(t)], e.want) for e, t in zip(entries, tokens_on_device)]
        return super().step(entries)


class AheadChooser(ArgmaxChooser):
    can_run_ahead = True
    unread = 0

    def choose_ahead(self, logits, sequence_indices):
        type(self).unread += 1
        assert type(self).unread <= 2               # the host is never more than one step behind
        return np.array(self.choose(logits, sequence_indices))

    def read(self, pending):
        type(self).unread -= 1
        return pending.tolist()

    def rows_of(self, pending, rows):
        return pending[list(rows)]


@pytest.mark.parametrize("kw", [dict(max_tokens=6, stop_ids=(23,)), dict(max_tokens=1), dict(max_tokens=2),
                                dict(max_tokens=40, ignore_eos=True), dict(max_tokens=3, ignore_eos=True)])
def test_decoding_one_step_ahead_of_the_host_gives_the_same(kw):
    """With an engine that takes tokens from the device and a chooser that leaves them there, the
    loop puts every decode step on the stream before it has read the tokens of the one before.
    Same tokens and stop reasons as step by step; a sequence that ends on a token's value has
    been through one step more (thrown away), one that ends by count or at the model's last
    position has not; every slot comes back."""
    prompts = [[5], [20, 21], [7, 8], [30, 31, 32]]
    params = SamplingParams(temperature=0.0, repeat_check=False, **kw)
    eng0 = FakeEngine()
    want = Generator(eng0, max_batch=4, make_chooser=ArgmaxChooser).generate(prompts, params)
    eng = AheadEngine()
    AheadChooser.unread = 0
    gen = Generator(eng, max_batch=4, make_chooser=AheadChooser)
    got = gen.generate(prompts, params)
    assert [(r.tokens, r.stop_reason) for r in got] == [(r.tokens, r.stop_reason) for r in want]
    assert eng.cache.slots.held_count == 0 and AheadChooser.unread == 0
    # what ran ahead for nothing: at most one step for every sequence that ended on a token's value
    by_value = sum(r.stop_reason in (EOS, STOP_TOKEN) for r in got)
    fed0 = sum(n for step in eng0.steps for _, n in step)
    fed = sum(n for step in eng.steps for _, n in step)
    assert fed0 <= fed <= fed0 + by_value
    if kw.get("ignore_eos"):
        assert fed == fed0                   # ends by count or position only: nothing is thrown away
    # the caller's word and the interrupt flag work one step behind as well
    eng = AheadEngine()
    AheadChooser.unread = 0
    res = Generator(eng, max_batch=4, make_chooser=AheadChooser).generate(
        prompts, SamplingParams(temperature=0.0, max_tokens=30, ignore_eos=True, repeat_check=False),
        on_token=lambda i, tok: "enough" if (i == 1 and tok == 25) else None,
        interrupt=lambda: len(eng.steps) >= 8)
    assert res[1].tokens == [22, 23, 24, 25] and res[1].stop_reason == "enough"
    assert all(r.stop_reason == INTERRUPTED for j, r in enumerate(res) if j != 1)
    assert eng.cache.slots.held_count == 0


def test_decoding_ahead_on_random_requests_gives_the_same():
    """Random prompts, stop tokens, budgets and batch sizes: the loop that runs one step ahead of
    the host and the step-by-step loop give the same results, and every slot comes back."""
    rng = random.Random(11)
    for trial in range(60):
        n = rng.randint(1, 9)
        prompts = [[rng.randrange(50) for _ in range(rng.randint(1, 6))] for _ in range(n)]
        params = SamplingParams(temperature=0.0, max_tokens=rng.choice([1, 2, 3, 7, 20, 60]),
                                stop_ids=tuple(rng.sample(range(50), rng.randint(0, 6))),
                                ignore_eos=rng.random() < 0.3, repeat_check=rng.random() < 0.5)
        max_batch = rng.choice([1, 2, 4, 16])
        want = Generator(FakeEngine(), max_batch=max_batch, make_chooser=ArgmaxChooser).generate(prompts, params)
        eng = AheadEngine()
        AheadChooser.unread = 0
        got = Generator(eng, max_batch=max_batch, make_chooser=AheadChooser).generate(prompts, params)
        assert [(r.tokens, r.stop_reason) for r in got] == [(r.tokens, r.stop_reason) for r in want], trial
        assert eng.cache.slots.held_count == 0 and AheadChooser.unread <= 1


# ---- a conversation: turns on a kept slot
class KeepingEngine(AheadEngine):
    """Remembers the tokens every slot holds, and can roll a slot back."""

    def __init__(self, ahead=True, rolls_back=True):
        super().__init__()
        self.accepts_device_tokens = ahead
        self.cache.rolls_back_freely = rolls_back
        self.held = {}
        self.rolled_back = 0

    def alloc_slot(self):
        s = super().alloc_slot()
        self.held[s] = []
        return s

    def step(self, entries, tokens_on_device=None):
        if any(len(e.tokens) > 1 for e in entries):
            AheadChooser.unread = 0          # a new turn: what ran ahead for nothing before it is forgotten
        if tokens_on_device is not None:
            entries = [type(e)(e.slot, [int(t)], e.want) for e, t in zip(entries, tokens_on_device)]
        for e in entries:
            self.held[e.slot].extend(e.tokens)
        return FakeEngine.step(self, entries)

    def truncate(self, slot, length):
        assert 0 <= length <= self.cache.lengths[slot]
        self.rolled_back += self.cache.lengths[slot] - length
        self.cache.lengths[slot] = length
        del self.held[slot][length:]


@pytest.mark.parametrize("ahead,rolls_back", [(False, True), (True, True), (True, False)])
def test_turns_on_a_kept_slot_go_on_from_what_it_holds(ahead, rolls_back):
    """Generator.extend: the slot is the caller's and is kept; after a turn it holds the turn's
    tokens and all generated ones but the newest, whether or not a step ran ahead of the host
    (the extra step is rolled back; where the cache cannot roll back nothing runs ahead)."""
    eng = KeepingEngine(ahead, rolls_back)
    AheadChooser.unread = 0
    gen = Generator(eng, max_batch=1, make_chooser=AheadChooser)
    chooser = AheadChooser(None, 1, 50, "cpu")
    slot = eng.alloc_slot()
    r1 = gen.extend(slot, [30, 31], SamplingParams(temperature=0.0, max_tokens=4, repeat_check=False), chooser)
    assert r1.tokens == [32, 33, 34, 35] and r1.stop_reason == MAX_TOKENS
    assert eng.held[slot] == [30, 31, 32, 33, 34] and eng.cache.length(slot) == 5
    # a turn that the model ends on a token's value: with a step ahead that token has been fed already
    r2 = gen.extend(slot, [35, 5], SamplingParams(temperature=0.0, max_tokens=10, repeat_check=False), chooser)
    assert r2.tokens == [6, 7, 8, 9] and r2.stop_reason == EOS
    assert eng.held[slot] == [30, 31, 32, 33, 34, 35, 5, 6, 7, 8] and eng.cache.length(slot) == 10
    assert eng.rolled_back == (1 if ahead and rolls_back else 0)
    # the caller's word ends a turn as well; the slot is still the caller's
    r3 = gen.extend(slot, [9, 40], SamplingParams(temperature=0.0, max_tokens=10, repeat_check=False), chooser,
                    on_token=lambda i, tok: "enough" if tok == 42 else None)
    assert r3.tokens == [41, 42] and r3.stop_reason == "enough" and eng.held[slot][-3:] == [9, 40, 41]
    assert eng.cache.slots.held_count == 1
    with pytest.raises(RequestError, match="does not fit"):
        gen.extend(slot, list(range(30)), SamplingParams(temperature=0.0, max_tokens=2), chooser)
    with pytest.raises(RequestError, match="at least one token"):
        gen.extend(slot, [], SamplingParams(temperature=0.0, max_tokens=2), chooser)
    eng.free_slot(slot)
    assert eng.cache.slots.held_count == 0


def test_decode_steps_run_at_a_ladder_of_sizes_filled_up_with_padding():
    """The fixed metadata of a decode step, without a GPU: a step of fewer sequences than its size
    is filled up with rows of one token (id 0, position 0) in the padding slot; the lists of ranges
    cover every row; how unequal the contexts are is judged on the sequences alone."""
    from herbert_rs_amd.engine.batch import StaticDecodeMeta, StepEntry, decode_batch_bucket, range_list
    ladder = [decode_batch_bucket(n) for n in range(1, 81)]
    assert ladder[:16] == [1, 2, 3, 4, 6, 6, 8, 8, 10, 10, 12, 12, 14, 14, 16, 16]
    assert sorted(set(ladder)) == [1, 2, 3, 4, 6, 8, 10, 12, 14, 16, 20, 24, 28, 32, 40, 48, 56, 64, 72, 80]
    assert [decode_batch_bucket(n) for n in (81, 129, 130, 257)] == [88, 144, 144, 288]
    assert all(b >= n and 4 * b <= 5 * n + 4 for n, b in enumerate(ladder, 1))      # within a quarter (and a row)
    meta = StaticDecodeMeta(6, "cpu", pad_slot=99)
    entries = [StepEntry(3, [11], [0]), StepEntry(7, [12], [0]), StepEntry(1, [13], [0]), StepEntry(2, [14], [0]),
               StepEntry(5, [15], [0])]
    m = meta.update(entries, [700, 9, 64, 0, 30])
    assert m.num_seqs == m.num_tokens == 6 and m.token_ids.tolist() == [11, 12, 13, 14, 15, 0]
    assert m.positions.tolist() == [700, 9, 64, 0, 30, 0] and m.slots.tolist() == [3, 7, 1, 2, 5, 99]
    assert m.context_lens.tolist() == [701, 10, 65, 1, 31, 1] and m.want_rows.tolist() == list(range(6))
    assert m.max_context == 701 and m.context_bucket == 768 and m.unequal == 2
    ranges = m.ranges_for(16, 64)           # five sequences and the padding row, each at least one range
    assert ranges.tolist() == range_list([701, 10, 65, 1, 31, 1], 16, 64).tolist() and ranges.tolist()[6] <= 16
    # the next step brings fewer sequences: the rows that held sequences are padding now
    m = meta.update(entries[:2], [701, 10])
    assert m.slots.tolist() == [3, 7, 99, 99, 99, 99] and m.context_lens.tolist() == [702, 11, 1, 1, 1, 1]
    assert m.token_ids.tolist()[2:] == [0, 0, 0, 0]
    with pytest.raises(ValueError, match="do not fit"):
        meta.update(entries + entries[:2], [1] * 7)


def test_the_memory_a_cache_needs_counts_pages_and_state():
    """What the engine compares with the GPU's free memory before it builds a cache: the pools of
    keys and values by pages, and fixed-size state by slots, entries of equal need together."""
    import torch
    from herbert_rs_amd.cache import Cache, KVNeed, StateNeed
    kv, state = KVNeed(2, 16, None), StateNeed((5, 8), torch.float32)
    needs = {0: kv, 1: (kv, state), 3: state}
    got = Cache.bytes_needed(needs, max_tokens=64 * 6 - 1, dtype=torch.bfloat16, max_slots=4)
    assert got == 2 * 2 * (6 + 1) * 64 * 2 * 16 * 2 + 2 * (4 + 1) * 40 * 4       # one page and one slot more: the padding's
    cache = Cache(needs, 64 * 6 - 1, 512, torch.bfloat16, "cpu", max_slots=4)
    held = sum(g.pool.numel() * 2 for g in cache.kv_groups.values()) + \
        sum(g.data.numel() * 4 for g in cache.state_groups.values())
    assert held == got
    # without a cap on the slots there are as many as pages
    assert Cache.bytes_needed({0: state}, 64 * 3, torch.float32) == (3 + 1) * 40 * 4


def test_a_token_that_is_none_ends_the_generation_with_an_error():
    """A chooser's -1 (the GPU argmax's answer for a row without a finite logit) is an error of the
    loop's, not a token; the slots still come back."""
    from herbert_rs_amd.errors import BackendError

    class NoneChooser(ArgmaxChooser):
        def choose(self, logits, sequence_indices):
            return [-1 for _ in sequence_indices]
    eng = FakeEngine()
    with pytest.raises(BackendError, match="no token could be chosen"):
        Generator(eng, max_batch=2, make_chooser=NoneChooser).generate(
            [[5], [6, 7]], SamplingParams(temperature=0.0, max_tokens=3, repeat_check=False))
    assert eng.cache.slots.held_count == 0


class CountingChooser(AheadChooser):
    """Counts the draws that each sequence's generator stream has given, as the GPU sampler's
    states advance once a choice."""

    def __init__(self, params, n, vocab, device):
        super().__init__(params, n, vocab, device)
        self.draws = [0] * n

    def choose(self, logits, sequence_indices):
        for i in sequence_indices:
            self.draws[i] += 1
        return super().choose(logits, sequence_indices)

    def save_streams(self):
        return list(self.draws)

    def restore_stream(self, sequence, saved):
        self.draws[sequence] = saved[sequence]


@pytest.mark.parametrize("ahead", [False, True])
def test_a_turn_on_a_kept_slot_takes_one_draw_a_token(ahead):
    """A turn that ends on a token's value has been through one step more when the loop runs ahead
    of the host, and that step has drawn from the sequence's generator: the draw is taken back,
    so that the next turn of a seeded conversation draws what it draws step by step. A turn that
    ends by count is not taken ahead and has nothing to take back."""
    eng = KeepingEngine(ahead, True)
    CountingChooser.unread = 0
    gen = Generator(eng, max_batch=1, make_chooser=CountingChooser)
    chooser = CountingChooser(None, 1, 50, "cpu")
    slot = eng.alloc_slot()
    r1 = gen.extend(slot, [35, 5], SamplingParams(temperature=0.0, max_tokens=10, repeat_check=False), chooser)
    assert r1.tokens == [6, 7, 8, 9] and r1.stop_reason == EOS
    assert eng.rolled_back == (1 if ahead else 0)
    assert chooser.draws == [4]
    CountingChooser.unread = 0           # (the step that ran ahead for nothing was never read)
    r2 = gen.extend(slot, [9, 20], SamplingParams(temperature=0.0, max_tokens=3, repeat_check=False), chooser)
    assert r2.tokens == [21, 22, 23] and r2.stop_reason == MAX_TOKENS and chooser.draws == [7]
    # a batch of the loop's own slots does not save anything: those streams end with their sequences
    CountingChooser.unread = 0
    got = Generator(AheadEngine(), max_batch=2, make_chooser=CountingChooser).generate(
        [[5], [30]], SamplingParams(temperature=0.0, max_tokens=6, repeat_check=False))
    assert [r.stop_reason for r in got] == [EOS, MAX_TOKENS]
    eng.free_slot(slot)


class WordTokenizer:
    """Words and the specials of a chat template as tokens; ids grow as words are first seen."""
    SPECIALS = ["<|im_start|>", "<|im_end|>", "\n"]

    def __init__(self):
        self.ids = {"<|im_start|>": 10, "<|im_end|>": 9, "\n": 11}

    def token_to_id(self, token):
        return self.ids.get(token)

    def encode(self, text, add_special_tokens=False):
        import re
        pieces = [p for p in re.split(r"(<\|im_start\|>|<\|im_end\|>|\n| )", text) if p and p != " "]
        for p in pieces:
            self.ids.setdefault(p, 12 + len(self.ids))
        return type("Encoding", (), {"ids": [self.ids[p] for p in pieces]})()

    def decode(self, ids, skip_special_tokens=True):
        names = {v: k for k, v in self.ids.items()}
        words = [names.get(i, f"#{i}") for i in ids]
        if skip_special_tokens:
            words = [w for w in words if w not in ("<|im_start|>", "<|im_end|>")]
        return " ".join(words)


def test_a_conversation_keeps_its_slot_and_runs_its_commands():
    """The chat loop with a stand-in engine (next token = last + 1, token 9 ends a turn) and a
    word tokenizer: what each turn feeds, the slash commands, a line continued with a backslash,
    /clear, the end of the input."""
    import io
    from herbert_rs_amd.chat import Chat, ChatSession
    from herbert_rs_amd.models.qwen3 import CHAT
    from herbert_rs_amd.sampling import ThinkTokens
    import herbert_rs_amd.chat as chat_mod

    class FakeSampler(AheadChooser):
        made = 0

        def __init__(self, params, n, vocab, device):
            super().__init__(params, n, vocab, device)
            type(self).made += 1
            self.turns = 0

        def new_turn(self):
            self.turns += 1

    import herbert_rs_amd.sampling.sampler as sampler_mod
    eng = KeepingEngine(ahead=True)
    eng.spec.max_positions = 200
    tok = WordTokenizer()
    params = SamplingParams(temperature=0.0, max_tokens=5, stop_ids=(9,), repeat_check=False)
    session = ChatSession(eng, tok, CHAT, params, system="be brief", end_id=9)
    lines = iter(["/config", "hello \\", "there", "/stats", "/temp 0.5", "/temp x", "/topk 7", "/topp 2", "/think 3",
                  "again", "/nope", "/clear", "/stats", "once more", "/tools", "", "/quit", "never read"])

    def read_line(prompt):
        try:
            return next(lines)
        except StopIteration:
            raise EOFError
    out, err = io.StringIO(), io.StringIO()
    real = sampler_mod.Sampler
    sampler_mod.Sampler = FakeSampler
    AheadChooser.unread = 0
    try:
        chat = Chat(session, think_tokens=lambda: ThinkTokens(20, 21, 11), read_line=read_line, out=out, err=err)
        assert chat.run() == 0
    finally:
        sampler_mod.Sampler = real
    said = err.getvalue()
    assert "--- Config (greedy) ---" in said and "think_budget: unlimited" in said
    assert "Usage: /temp <value>" in said and "Top-p must be between 0 and 1" in said
    assert "think_budget: 3 tokens" in said and "Unknown command: /nope" in said
    assert "[Conversation cleared]" in said and "KV cache tokens: 0 (cleared)" in said
    assert "/tools is not available here" in said and "Turns:           1" in said
    assert next(lines) == "never read"                       # /quit ended the loop
    assert eng.cache.slots.held_count == 0                   # the slot went back at the end
    # the first turn: the template with the system prompt, the two lines joined by a line break
    first = tok.encode(CHAT.build_prompt("hello \nthere", "be brief")).ids
    assert session.turns == 3 and FakeSampler.made == 2      # the commands that change parameters made a new sampler, /clear none
    # what the slots held is gone with them; the turns' tokens are seen in the steps' sizes
    sizes = [n for step in eng.steps for _, n in step]
    assert sizes[0] == len(first)
    # the model's text went to `out`, one line a turn
    assert len(out.getvalue().strip().split("\n")) == 3


def test_a_turn_begins_with_the_token_the_last_one_ended_on():
    from herbert_rs_amd.chat import ChatSession
    from herbert_rs_amd.models.qwen3 import CHAT
    import herbert_rs_amd.sampling.sampler as sampler_mod

    class FakeSampler(AheadChooser):
        def new_turn(self):
            pass
    real = sampler_mod.Sampler
    sampler_mod.Sampler = FakeSampler
    AheadChooser.unread = 0
    try:
        eng = KeepingEngine(ahead=True)
        eng.spec.max_positions = 300
        tok = WordTokenizer()
        tok.ids.update({"a": 5, "b": 30})
        session = ChatSession(eng, tok, CHAT, SamplingParams(temperature=0.0, max_tokens=3, stop_ids=(9,),
                                                              repeat_check=False), end_id=9)
        # "assistant" and the line break that ends the template get ids 12.. ; the reply counts on from the last
        r1 = session.say("a")
        slot = session.slot
        held1 = list(eng.held[slot])
        assert held1[:-len(r1.tokens) + 1 or None][:len(tok.encode(CHAT.build_prompt("a", None)).ids)] == \
            tok.encode(CHAT.build_prompt("a", None)).ids
        assert r1.stop_reason == MAX_TOKENS and session.last_token == r1.tokens[-1]
        assert held1 == tok.encode(CHAT.build_prompt("a", None)).ids + r1.tokens[:-1]
        # cut short: the next turn brings the last token, the end-of-turn token, the line break, the template
        r2 = session.say("b")
        want = held1 + [r1.tokens[-1], 9, 11] + tok.encode(CHAT.build_prompt("b", None)).ids + r2.tokens[:-1]
        assert eng.held[slot] == want
        # a turn that the model ended itself: its last token is the end-of-turn token and is not doubled
        session.last_token = 9
        assert session.turn_tokens("b")[:3] == [9, 11, 10]
        # no room: the turn is refused and the conversation is still there
        eng.spec.max_positions = len(want) + 5
        with pytest.raises(RequestError, match="no room left"):
            session.say("b")
        assert session.slot == slot
        session.clear()
        assert eng.cache.slots.held_count == 0
    finally:
        sampler_mod.Sampler = real


def test_command_line_pieces_that_need_no_gpu(tmp_path, capsys):
    """What the command line decides before it loads a model: stop strings unescaped and
    searched in the text's tail (crates/cli/src/main.rs:212-258), token ids parsed
    (crates/cli/src/token_parser.rs:13-26), no conversation without a tokenizer, the text of a
    stream printed once and never with a trailing replacement character."""
    import io
    import json
    from herbert_rs_amd import cli
    from .tiny import TINY_A
    assert cli.decode_escaped_text(r"a\nb\t\\c\q\0") == "a\nb\t\\c\\q\0"
    assert cli.normalize_stop_sequences([" x ", "x", "", r"\n\n"]) == ["x", "\n\n"]
    assert cli.find_stop_sequence("so it ends. END", ["never", "END"]) == "END"
    assert cli.find_stop_sequence("END" + "." * 200, ["END"]) is None          # only the tail is searched
    assert cli.parse_token_ids("5, 17,3") == [5, 17, 3]
    with pytest.raises(RequestError, match="Invalid token ID"):
        cli.parse_token_ids("5,x")
    with pytest.raises(RequestError, match="Need tokenizer.json"):
        cli.parse_token_ids("hello")
    folder = tmp_path / "m"
    folder.mkdir()
    (folder / "config.json").write_text(json.dumps(TINY_A))
    assert cli.main(["--model", str(folder)]) == 1
    assert "the conversation needs a tokenizer.json" in capsys.readouterr().err
    assert cli.main([]) == 1 and "--model is required" in capsys.readouterr().err
    # one backend under two names, as the reference lists its own (crates/cli/src/main.rs:367-386)
    assert cli.main(["--backend", "help"]) == 0 and cli.BACKEND in capsys.readouterr().err
    assert cli.main(["--backend", "metal", "--model", str(folder)]) == 1
    assert "unknown backend 'metal'" in capsys.readouterr().err
    assert cli.main(["--gpu", "x", "--model", str(folder)]) == 1
    assert '--gpu must be a number or "list"' in capsys.readouterr().err
    assert cli.main(["--gpu", "7", "--model", str(folder)]) == 1 and "--gpu 7" in capsys.readouterr().err
    assert cli.main(["--gpu", "list"]) == 0

    class Pieces:
        """Token 1 is the first half of a character, token 2 its second half."""
        def decode(self, ids, skip_special_tokens=True):
            text = ""
            for a, b in zip(ids[::2], ids[1::2] + [None]):
                text += "é" if (a, b) == (1, 2) else ("�" if b is None and a == 1 else f"<{a}>" + (f"<{b}>" if b else ""))
            return text
    out = io.StringIO()
    printer = cli.StreamPrinter(Pieces(), out=out, stop_strings=["é"])
    assert printer.on_token(0, 1) is None and out.getvalue() == ""             # half a character: nothing yet
    assert printer.on_token(0, 2) == STOP_SEQUENCE and out.getvalue() == "é"
    ids_out = io.StringIO()
    plain_printer = cli.StreamPrinter(None, out=ids_out)
    plain_printer.on_token(0, 7), plain_printer.on_token(0, 8)
    assert ids_out.getvalue() == "7,8"


def test_replay_reads_steps_and_names_what_is_wrong_with_them(tmp_path):
    """The replay program's reading of its input, with a stand-in engine: slots by request id,
    given back at "end", logits written for the steps that want some, clear errors for a step
    that is no such object and for a request that ends without having started."""
    from herbert_rs_amd.engine.replay import Replayer

    class Rows:
        def __init__(self, a):
            self.a = a

        def detach(self):
            return self

        def to(self, _):
            return self

        def numpy(self):
            return self.a

    class Eng(FakeEngine):
        def step(self, entries):
            out = super().step(entries)
            return None if out is None else Rows(out)
    eng = Eng()
    rp = Replayer(eng, str(tmp_path / "out"))
    assert rp.run_step({"step": 0, "entries": [{"id": "a", "tokens": [5, 6], "want": [1]},
                                               {"id": "b", "tokens": [9], "want": []}], "end": []}) == 0
    got = np.fromfile(tmp_path / "out" / "0.f32", dtype="<f4").reshape(1, -1)
    assert got.shape == (1, 50) and got[0].argmax() == 7
    assert rp.run_step({"step": 1, "entries": [{"id": "a", "tokens": [7]}], "end": ["b"]}) == 1
    assert not (tmp_path / "out" / "1.f32").exists() and eng.cache.slots.held_count == 1
    assert eng.steps == [[(0, 2), (1, 1)], [(0, 1)]]
    with pytest.raises(RequestError, match="ends but never started"):
        rp.run_step({"step": 2, "entries": [], "end": ["zz"]})
    for bad in ({"entries": []}, {"step": 3, "entries": [{"tokens": [1]}]}, {"step": 3, "entries": [{"id": "c", "tokens": ["x"]}]},
                {"step": 3, "entries": 7}):
        with pytest.raises(RequestError, match="a step is an object"):
            rp.run_step(bad)
    assert rp.run_step({"step": 4, "entries": [], "end": ["a"]}) == 4 and eng.cache.slots.held_count == 0


def test_lists_of_ranges_cover_every_sequence_and_follow_the_steps():
    """The list that deals a decode grid out over sequences of unequal lengths: every sequence's
    ranges cover its pages, none has a range too many, all together fit the grid, with the shortest
    ranges that do; a step with fixed
    buffers makes its lists again at every update; what counts as unequal."""
    from herbert_rs_amd.engine.batch import StaticDecodeMeta, StepEntry, unequal_level, pack, range_list
    rng = random.Random(5)
    for _ in range(300):
        B = rng.randint(1, 64)
        items = rng.randint(B + 1, 4 * B + 8)
        unit = rng.choice([16, 64])
        ctx = [rng.choice([1, unit - 1, unit, unit + 1, rng.randint(1, 40000)]) for _ in range(B)]
        got = range_list(ctx, items, unit)
        per, counts = int(got[B + 1]), np.diff(got[:B + 1])
        assert got[0] == 0 and got[B] <= items and per >= 1 and (counts >= 1).all()
        for n, c in zip(ctx, counts):
            pages = -(-n // unit)
            assert (c - 1) * per < pages <= c * per
        # and no shorter range would do
        assert per == 1 or sum(-(-(-(-n // unit)) // (per - 1)) for n in ctx) > items
    with pytest.raises(ValueError):
        range_list([5, 5], 2, 64)
    assert [unequal_level(c) for c in ([700], [500, 500, 501], [1000, 300], [4096] + [2048] * 3)] == [0, 0, 0, 0]
    assert [unequal_level(c) for c in ([1000, 100], [1000, 50, 500], [4096] + [1024] * 7)] == [1, 1, 2]
    assert [unequal_level(c) for c in ([1000, 1, 1], [32768] + [1024] * 7, [8192] + [512] * 127)] == [2, 2, 2]

    static = StaticDecodeMeta(3, torch.device("cpu"))
    entries = [StepEntry(4, [7], [0]), StepEntry(2, [8], [0]), StepEntry(9, [9], [0])]
    meta = static.update(entries, [5000, 10, 63])
    assert meta.unequal and list(meta.host_context) == [5001, 11, 64]
    first = meta.ranges_for(16, 64)
    assert first.tolist() == range_list([5001, 11, 64], 16, 64).tolist()
    assert meta.ranges_for(16, 64) is first                  # one list for all who ask for the same
    other = meta.ranges_for(8, 64)
    meta = static.update(entries, [5055, 64, 64])            # a page more for each
    assert first.tolist() == range_list([5056, 65, 65], 16, 64).tolist()
    assert other.tolist() == range_list([5056, 65, 65], 8, 64).tolist()
    assert meta.ranges_for(16, 64) is first
    for items in (32, 64):
        assert meta.ranges_for(items, 64) is not None
    assert meta.ranges_for(128, 64) is None                  # no room for a fifth list: the caller does without
    meta = static.update(entries, [70, 64, 64])
    assert not meta.unequal and list(meta.slots) == [4, 2, 9]
    meta = static.update(entries, [900, 65, 65])               # unequal again: the lists follow
    assert meta.unequal and first.tolist() == range_list([901, 66, 66], 16, 64).tolist()

    packed = pack(entries, [5000, 10, 63], torch.device("cpu"))
    assert packed.unequal and packed.ranges_for(16, 64).tolist() == range_list([5001, 11, 64], 16, 64).tolist()
    assert not pack(entries, [64, 10, 63], torch.device("cpu")).unequal


def test_context_buckets_grow_with_the_context():
    """What sizes the decode kernels' grids and names a captured graph: multiples of 256 up to
    4,096 tokens, then eight buckets for every doubling; never below the context, never more than
    an eighth above it beyond the first buckets."""
    from herbert_rs_amd.engine.batch import bucket
    assert [bucket(c) for c in (1, 256, 257, 4096, 4097, 4608, 4609, 8192, 8193, 16384, 16385, 32768)] == \
        [256, 256, 512, 4096, 4608, 4608, 5120, 8192, 9216, 16384, 18432, 32768]
    assert len({bucket(c) for c in range(1, 32769)}) == 16 + 8 + 8 + 8
    for c in list(range(1, 10000, 37)) + [40000, 131072, 131073, 1000000]:
        assert c <= bucket(c) < max(c + 256, c * 9 // 8)
