"""Schedules beyond a batch that starts together: a step that carries running sequences' single
tokens beside a new sequence's whole prompt, a roll-back followed by other tokens, a step that
does not fit, checkpoints with tensors nobody asks for, many decode graphs, stop strings."""
import json
import os
import signal
import subprocess
import sys
import time

import numpy as np
import pytest
import torch

import herbert_rs_amd as hb
from herbert_rs_amd.engine import StepEntry
from herbert_rs_amd.errors import CacheError

from .bounds import close
from .plain import model as plain
from .plain_cache import plain_folder, plain_logits
from .tiny import CONFIGS, make_folder, random_tokens

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["B", "D"])
def test_decoding_sequences_and_a_new_prompt_in_one_step(name, dtype, model_root):
    """Continuous batching's shape: two sequences that have run for a while bring one token each,
    in the same step as the whole prompt of a sequence that starts, and as a piece of a prompt that
    was begun before. Every logit is the one the sequence gets alone."""
    folder = make_folder(model_root, name, dtype)
    raw = CONFIGS[name][0]
    vocab = raw["vocab_size"]
    long_n = 200 if name == "B" else 900
    a, b = random_tokens(vocab, long_n + 6, 201), random_tokens(vocab, 70 + 6, 202)
    c, d = random_tokens(vocab, 97 + 3, 203), random_tokens(vocab, 130, 204)
    ref = {k: plain_logits(folder, t) for k, t in (("a", a), ("b", b), ("c", c), ("d", d))}
    engine = hb.load(folder, dtype=dtype, cache_tokens=64 * 40)
    sa, sb = engine.alloc_slot(), engine.alloc_slot()
    engine.step([StepEntry(sa, a[:long_n], []), StepEntry(sb, b[:70], [])])
    for p in range(3):                                              # both decode for a while
        engine.step([StepEntry(sa, [a[long_n + p]], [0]), StepEntry(sb, [b[70 + p]], [0])])
    sc, sd = engine.alloc_slot(), engine.alloc_slot()
    engine.step([StepEntry(sd, d[:40], [])])                         # d's prompt has begun
    # the mixed step: a and b one token each, c whole, d's next piece
    got = engine.step([StepEntry(sa, [a[long_n + 3]], [0]), StepEntry(sc, c[:97], [0, 50, 96]),
                       StepEntry(sb, [b[73]], [0]), StepEntry(sd, d[40:110], [0, 69])]).cpu().numpy()
    want = [("a", long_n + 3), ("c", 0), ("c", 50), ("c", 96), ("b", 73), ("d", 40), ("d", 109)]
    for row, (k, p) in enumerate(want):
        ok, err = close(got[row], ref[k][p], dtype, name, "mixed step")
        assert ok, (k, p, err)
    # and all four go on, one token each, from what that step left in the cache
    got = engine.step([StepEntry(sa, [a[long_n + 4]], [0]), StepEntry(sb, [b[74]], [0]),
                       StepEntry(sc, [c[97]], [0]), StepEntry(sd, [d[110]], [0])]).cpu().numpy()
    for row, (k, p) in enumerate([("a", long_n + 4), ("b", 74), ("c", 97), ("d", 110)]):
        ok, err = close(got[row], ref[k][p], dtype, name, "after mixed step")
        assert ok, (k, p, err)
    for s in (sa, sb, sc, sd):
        engine.free_slot(s)
    engine.cache.check()


@pytest.mark.parametrize("name,lengths", [("D", [1780, 3, 70, 250, 64]), ("F", [3050, 10, 500, 64, 129, 1, 63, 700])])
def test_decoding_a_batch_of_very_unequal_lengths(name, lengths, model_root):
    """One long sequence beside short ones, decoded together for 40 steps: the attention deals its
    grid out by a list of ranges that the host makes again at every step (sequences pass the ends
    of pages and of context buckets on the way, the first step runs eagerly, the second is
    captured, the rest are replays), and the shortest sequence ends earlier. Every logit is the one
    the sequence gets alone."""
    folder = make_folder(model_root, name, "bfloat16")
    raw = CONFIGS[name][0]
    vocab = raw["vocab_size"]
    steps = 40
    toks = [random_tokens(vocab, n + (steps if i != 1 else 9), 700 + i) for i, n in enumerate(lengths)]
    ref = [plain_logits(folder, t) for t in toks]
    engine = hb.load(folder, dtype="bfloat16", cache_tokens=64 * (sum(-(-(n + steps) // 64) for n in lengths) + 2))
    slots = [engine.alloc_slot() for _ in lengths]
    engine.step([StepEntry(s, t[:n], []) for s, t, n in zip(slots, toks, lengths)])
    live = list(range(len(lengths)))
    for j in range(steps):
        live = [i for i in live if lengths[i] + j < len(toks[i])]
        got = engine.step([StepEntry(slots[i], [toks[i][lengths[i] + j]], [0]) for i in live]).cpu().numpy()
        for row, i in enumerate(live):
            ok, err = close(got[row], ref[i][lengths[i] + j], "bfloat16", name, "unequal batch")
            assert ok, (i, j, err)
    items = 1024 // raw["num_key_value_heads"]
    from herbert_rs_amd.engine.batch import decode_batch_bucket
    for B in {decode_batch_bucket(len(lengths)), decode_batch_bucket(len(lengths) - 1)}:      # (the steps' sizes)
        assert engine._decode[B].static.range_lists == [(items, 64)]      # the list was what ran
    assert engine.graphs_captured >= 2          # (a context bucket's edge is passed on the way)
    for s in slots:
        engine.free_slot(s)
    engine.cache.check()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["B", "D"])
def test_roll_back_and_feed_other_tokens(name, dtype, model_root):
    """Engine.truncate (the reference's truncate_kv, crates/backends/backend_common/src/
    cpu_backend.rs:527-543): 150 tokens, back to 70 (inside a page: the rest of that page holds
    keys and, transposed, values of the tokens given up) and to 64 (a page's edge), then other
    tokens, whole and one by one; every position's logits are those of the new sequence."""
    folder = make_folder(model_root, name, dtype)
    vocab = CONFIGS[name][0]["vocab_size"]
    first = random_tokens(vocab, 150, 301)
    engine = hb.load(folder, dtype=dtype, cache_tokens=64 * 8)
    group = next(iter(engine.cache.kv_groups.values()))
    for keep, seed in ((70, 302), (64, 303), (0, 304), (149, 305)):
        s = engine.alloc_slot()
        engine.step([StepEntry(s, first, [])])
        assert group.pages.held_count == 3
        engine.truncate(s, keep)
        assert engine.cache.length(s) == keep and group.pages.held_count == (keep + 63) // 64
        other = first[:keep] + random_tokens(vocab, 60, seed)
        ref = plain_logits(folder, other)
        got = [engine.step([StepEntry(s, other[keep:keep + 30], list(range(30)))]).cpu().numpy()]
        for p in range(keep + 30, keep + 60):
            got.append(engine.step([StepEntry(s, [other[p]], [0])]).cpu().numpy())
        got = np.concatenate(got)
        for i, p in enumerate(range(keep, keep + 60)):
            ok, err = close(got[i], ref[p], dtype, name, "after roll-back")
            assert ok, (keep, p, err)
        with pytest.raises(CacheError, match="cannot truncate"):
            engine.truncate(s, keep + 61)
        engine.free_slot(s)
        engine.cache.check()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["C", "D"])
def test_turns_on_a_kept_slot_leave_the_whole_conversation_in_the_cache(name, dtype, model_root):
    """Generator.extend, the conversation's step (the reference's continue_prefill and decode on a
    kept KvHandle, crates/cli/src/chat.rs:1060-1075): three turns on one slot, each ended by a
    word of the caller's (where a step ran ahead of the host it is rolled back; the windowed
    configuration C cannot roll back and runs nothing ahead). Afterwards the slot holds
    every turn's tokens and all generated ones but the newest, and the logits of the next tokens
    are those of the plain model on that whole sequence."""
    from herbert_rs_amd.engine.generate import Generator
    from herbert_rs_amd.sampling import SamplingParams
    from herbert_rs_amd.sampling.sampler import Sampler
    folder = make_folder(model_root, name, dtype)
    vocab = CONFIGS[name][0]["vocab_size"]
    engine = hb.load(folder, dtype=dtype, cache_tokens=64 * 8)
    assert engine.cache.rolls_back_freely == (name == "D")
    gen = Generator(engine, max_batch=1, prefill_chunk=40)
    slot = engine.alloc_slot()
    sequence, last = [], []
    for turn, n in enumerate((70, 3, 58)):
        tokens = last + random_tokens(vocab, n, 400 + turn)
        # the caller ends the turn at its third token: nobody knew beforehand that it would end there
        params = SamplingParams(temperature=0.0, max_tokens=6, ignore_eos=True, repeat_check=False)
        said = []
        r = gen.extend(slot, tokens, params, Sampler(params, 1, vocab, engine.device),
                       on_token=lambda i, t: said.append(t) or ("enough" if len(said) == 3 else None))
        assert r.tokens == said and len(said) == 3 and r.stop_reason == "enough"
        sequence += tokens + r.tokens[:-1]
        last = [r.tokens[-1]]
        assert engine.cache.length(slot) == len(sequence)
    more = last + random_tokens(vocab, 9, 410)
    ref = plain_logits(folder, sequence + more)
    got = engine.step([StepEntry(slot, more, list(range(len(more))))]).cpu().numpy()
    for i in range(len(more)):
        ok, err = close(got[i], ref[len(sequence) + i], dtype, name, "after three turns")
        assert ok, (i, err)
    engine.free_slot(slot)
    engine.cache.check()


def test_seeded_turns_draw_the_same_with_and_without_a_step_ahead(model_root):
    """A seeded conversation at temperature 0.8 whose sampler goes on from turn to turn: with decode
    steps put on the stream one ahead of the host, a turn that ends on a token's value has drawn once
    more than it has tokens; the draw is taken back, so that every turn's tokens and the generator's
    state after it are those of the loop that waits for each token (one draw a token, as the
    reference's sampler draws)."""
    from herbert_rs_amd.engine.generate import Generator
    from herbert_rs_amd.sampling import SamplingParams
    from herbert_rs_amd.sampling.sampler import Sampler
    folder = make_folder(model_root, "D", "float32")
    vocab = CONFIGS["D"][0]["vocab_size"]
    turns = [random_tokens(vocab, n, 430 + i) for i, n in enumerate((30, 4, 17))]
    outcome = {}
    for ahead in (False, True):
        engine = hb.load(folder, dtype="float32", cache_tokens=64 * 6)
        gen = Generator(engine, max_batch=1, run_ahead=ahead)
        params = SamplingParams(temperature=0.8, top_k=20, top_p=1.0, max_tokens=12, ignore_eos=True,
                                repeat_check=False, seed=5)
        sampler = Sampler(params, 1, vocab, engine.device)
        slot = engine.alloc_slot()
        said, states, last = [], [], []
        for turn, tokens in enumerate(turns):
            count = []
            # the caller ends the turn at its fifth token: a value nobody knew beforehand
            r = gen.extend(slot, last + tokens, params, sampler,
                           on_token=lambda i, t: count.append(t) or ("enough" if len(count) == 5 else None))
            assert len(r.tokens) == 5
            said.append(r.tokens)
            states.append(int(sampler.states[0].item()))
            last = [r.tokens[-1]]
        outcome[ahead] = (said, states)
        engine.free_slot(slot)
        engine.cache.check()
    assert outcome[True] == outcome[False]
    # five draws a turn: the state after the turns is the seed's stream stepped 5, 10 and 15 times
    from herbert_rs_amd.sampling import xorshift
    state, want = xorshift.initial_state(5), []
    for n in range(15):
        state = xorshift.step(state)
        if n % 5 == 4:
            want.append(state - (1 << 64) if state >= (1 << 63) else state)
    assert outcome[True][1] == want


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_windowed_cache_rolls_back_only_to_keys_it_still_has(dtype, model_root):
    """Configuration C: one layer sees 70 keys and has given up the pages before them. Rolling
    back a little stays within what is held and gives the plain logits; rolling back past it is
    refused and changes nothing."""
    folder = make_folder(model_root, "C", dtype)
    vocab = CONFIGS["C"][0]["vocab_size"]
    first = random_tokens(vocab, 200, 311)
    engine = hb.load(folder, dtype=dtype, cache_tokens=64 * 8)
    s = engine.alloc_slot()
    engine.step([StepEntry(s, first, [])])
    with pytest.raises(CacheError, match="given up"):
        engine.truncate(s, 100)
    assert engine.cache.length(s) == 200
    engine.cache.check()
    # after 200 tokens the windowed layer holds pages from position 128 on; a query at 198 sees
    # the keys from 129 on
    with pytest.raises(CacheError, match="given up"):
        engine.truncate(s, 196)
    engine.truncate(s, 198)
    other = first[:198] + random_tokens(vocab, 20, 312)
    ref = plain_logits(folder, other)
    got = engine.step([StepEntry(s, other[198:], list(range(20)))]).cpu().numpy()
    for i in range(20):
        ok, err = close(got[i], ref[198 + i], dtype, "C", "after roll-back")
        assert ok, (i, err)
    engine.free_slot(s)
    engine.cache.check()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_window_with_heads_of_128(dtype, model_root):
    """Configuration D with a window of 100 keys on its first layer: in bfloat16 the window goes
    through the matrix-core attention of prompts (tiles whose first pages are out of sight) and
    through the decode kernel that norms, rotates and writes the cache itself, while the windowed
    layer's cache gives pages back; prompts of unequal lengths in one step, then one token each
    across page edges."""
    over = {"sliding_window": 100, "layer_types": ["sliding_attention", "full_attention"]}
    folder = make_folder(model_root, "D", dtype, overrides=over)
    vocab = CONFIGS["D"][0]["vocab_size"]
    seqs = [random_tokens(vocab, n + 70, 400 + n) for n in (300, 31, 130)]
    cuts = [300, 31, 130]
    refs = [plain_logits(folder, t) for t in seqs]
    engine = hb.load(folder, dtype=dtype, cache_tokens=64 * 12)
    windowed = [g for need, g in engine.cache.kv_groups.items() if need.window][0]
    slots = [engine.alloc_slot() for _ in seqs]
    got = engine.step([StepEntry(s, t[:c], [0, c // 2, c - 1]) for s, t, c in zip(slots, seqs, cuts)]).cpu().numpy()
    for i, c in enumerate(cuts):
        for j, p in enumerate((0, c // 2, c - 1)):
            ok, err = close(got[3 * i + j], refs[i][p], dtype, "D", "window")
            assert ok, (i, p, err)
    for k in range(70):
        got = engine.step([StepEntry(s, [t[c + k]], [0]) for s, t, c in zip(slots, seqs, cuts)]).cpu().numpy()
        for i, c in enumerate(cuts):
            ok, err = close(got[i], refs[i][c + k], dtype, "D", "window")
            assert ok, (i, c + k, err)
    assert windowed.first_page[slots[0]] == (370 + 1 - 100) // 64       # pages out of every later query's sight are back
    for s in slots:
        engine.free_slot(s)
    engine.cache.check()


@pytest.mark.parametrize("dtype", ["bfloat16", "float32"])
def test_long_prompts_take_the_kernel_for_them_by_themselves(dtype, model_root):
    """Configuration F (eight kv heads): a step of 4,100 prompt tokens has 520 attention workgroups
    of 64-token tiles, from which on the host takes the kernel for long prompts (two halves of 32
    tokens share a tile's pages); nothing is asked for by name. Two prompts of unequal lengths in
    the step, one of them going on from 37 tokens already in the cache (its tiles start at
    positions that 64 does not divide, and its last tile has 27 rows: one half is short), then
    single tokens."""
    from herbert_rs_amd.kernels import mfma
    folder = make_folder(model_root, "F", dtype)
    vocab = CONFIGS["F"][0]["vocab_size"]
    a, b = random_tokens(vocab, 2600 + 4, 501), random_tokens(vocab, 37 + 1500 + 4, 502)
    ref_a, ref_b = plain_logits(folder, a), plain_logits(folder, b)
    engine = hb.load(folder, dtype=dtype, cache_tokens=64 * 70)
    sa, sb = engine.alloc_slot(), engine.alloc_slot()
    engine.step([StepEntry(sb, b[:37], [])])
    entries = [StepEntry(sa, a[:2600], [0, 31, 32, 63, 64, 1300, 2559, 2560, 2599]),
               StepEntry(sb, b[37:1537], [0, 26, 27, 700, 1472, 1473, 1499])]
    meta_tiles = -(-2600 // 64) + -(-1500 // 64)
    assert meta_tiles * 8 >= mfma.PREFILL_LONG_MIN_WORKGROUPS
    got = engine.step(entries).cpu().numpy()
    row = 0
    for ref, base, e in ((ref_a, 0, entries[0]), (ref_b, 37, entries[1])):
        for p in e.want:
            ok, err = close(got[row], ref[base + p], dtype, "F", "long prompt")
            assert ok, (base + p, err)
            row += 1
    for k in range(4):
        got = engine.step([StepEntry(sa, [a[2600 + k]], [0]), StepEntry(sb, [b[1537 + k]], [0])]).cpu().numpy()
        assert close(got[0], ref_a[2600 + k], dtype, "F", "long prompt")[0]
        assert close(got[1], ref_b[1537 + k], dtype, "F", "long prompt")[0]
    engine.free_slot(sa)
    engine.free_slot(sb)
    engine.cache.check()


def test_a_step_that_does_not_fit_changes_nothing(model_root):
    """All of a step's pages or none: the step is refused, the sequences that were in it hold
    what they held, and they go on as if it had never been asked for."""
    folder = make_folder(model_root, "B", "float32")
    vocab = CONFIGS["B"][0]["vocab_size"]
    a, b = random_tokens(vocab, 80, 321), random_tokens(vocab, 140, 322)
    engine = hb.load(folder, dtype="float32", cache_tokens=64 * 4)
    sa, sb = engine.alloc_slot(), engine.alloc_slot()
    engine.step([StepEntry(sa, a[:60], []), StepEntry(sb, b[:10], [])])
    group = next(iter(engine.cache.kv_groups.values()))
    held = group.pages.held_count
    with pytest.raises(CacheError, match="more pages"):
        engine.step([StepEntry(sa, a[60:70], [9]), StepEntry(sb, b[10:140], [0])])   # 1 + 2 pages, 2 free
    assert group.pages.held_count == held
    assert engine.cache.length(sa) == 60 and engine.cache.length(sb) == 10
    engine.cache.check()
    got = engine.step([StepEntry(sa, a[60:80], [19]), StepEntry(sb, b[10:64], [53])]).cpu().numpy()
    assert close(got[0], plain_logits(folder, a)[79], "float32", "B")[0]
    assert close(got[1], plain_logits(folder, b)[63], "float32", "B")[0]
    engine.free_slot(sa)
    engine.free_slot(sb)
    engine.cache.check()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_checkpoint_with_tensors_nobody_asks_for_loads_and_says_the_same(dtype, model_root, tmp_path):
    """A tied model whose file also holds a head and rotary buffers (as exported checkpoints do):
    the reference ignores what it does not know and takes the embedding for the head
    (crates/backends/backend_common/src/loader_common.rs:679-685,1851-1872). Same logits as
    without them; the engine says what it passed over."""
    from safetensors.torch import load_file, save_file
    src = make_folder(model_root, "A", dtype)
    tensors = load_file(os.path.join(src, "model.safetensors"))
    tensors["lm_head.weight"] = torch.full((256, 64), 3.0).to(tensors["model.norm.weight"].dtype)
    for layer in range(2):
        tensors[f"model.layers.{layer}.self_attn.rotary_emb.inv_freq"] = torch.ones(8)
    save_file(tensors, str(tmp_path / "model.safetensors"))
    with open(os.path.join(src, "config.json")) as f, open(tmp_path / "config.json", "w") as g:
        g.write(f.read())
    tokens = random_tokens(256, 40, 331)
    engine = hb.load(str(tmp_path), dtype=dtype, cache_tokens=64)
    assert sorted(engine.ignored_tensors) == ["lm_head.weight", "model.layers.0.self_attn.rotary_emb.inv_freq",
                                              "model.layers.1.self_attn.rotary_emb.inv_freq"]
    s = engine.alloc_slot()
    got = engine.step([StepEntry(s, tokens, list(range(40)))]).cpu().numpy()
    clean = hb.load(src, dtype=dtype, cache_tokens=64)
    s2 = clean.alloc_slot()
    assert np.array_equal(got, clean.step([StepEntry(s2, tokens, list(range(40)))]).cpu().numpy())
    ref = plain_logits(src, tokens)
    for p in range(40):
        assert close(got[p], ref[p], dtype, "A")[0], p


def test_decode_graphs_and_their_logits_are_bounded(model_root, monkeypatch):
    """Decoding at three batch sizes up to 5,124 tokens of context, through 19 context buckets each
    (of 256 tokens up to 4,096, of 512 beyond): 57 shapes, more than the engine keeps graphs for (here 48). One logits buffer for all of them, at most MAX_GRAPHS
    graphs, the memory held levels off, and a shape whose graph was dropped is captured again and
    still says what eager steps say."""
    from herbert_rs_amd.engine import engine as eng_mod
    monkeypatch.setattr(eng_mod, "MAX_GRAPHS", 48)
    folder = make_folder(model_root, "D", "bfloat16", overrides={"max_position_embeddings": 8192})
    vocab = CONFIGS["D"][0]["vocab_size"]
    sizes = (1, 3, 8)
    engine = hb.Engine.from_folder(folder, dtype="bfloat16", max_tokens=64 * 90 * 8, use_graphs=True)
    eager = hb.Engine.from_folder(folder, dtype="bfloat16", max_tokens=64 * 90 * 8, use_graphs=False)
    feed = random_tokens(vocab, 8 * 64, 341)
    held_after = []
    for B in sizes:
        slots = [engine.alloc_slot() for _ in range(B)]
        slots_e = [eager.alloc_slot() for _ in range(B)]
        at = 0
        for bucket in range(20):
            grow = 256 * bucket + 250 - at                    # up to just below the next bucket's edge
            for eng, sl in ((engine, slots), (eager, slots_e)):
                eng.step([StepEntry(s, [(7 * i + j) % vocab for j in range(grow)], []) for i, s in enumerate(sl)])
            at += grow
            for j in range(10):                                # 6 steps in this bucket, 4 in the next
                toks = [feed[(at + 13 * i + j) % len(feed)] for i in range(B)]
                a = engine.step([StepEntry(s, [t], [0]) for s, t in zip(slots, toks)]).cpu().numpy()
                b = eager.step([StepEntry(s, [t], [0]) for s, t in zip(slots_e, toks)]).cpu().numpy()
                assert np.array_equal(a, b), (B, bucket, j)
                at += 1
        for s in slots:
            engine.free_slot(s)
        for s in slots_e:
            eager.free_slot(s)
        torch.cuda.synchronize()
        held_after.append(torch.cuda.memory_allocated())
    assert held_after[-1] - held_after[0] < 64 << 20           # no pool of its own behind every graph
    graphs, batch_sizes, logits_bytes = engine.decode_graph_stats()
    assert engine.graphs_captured >= 3 * 19                    # every shape was captured once
    assert graphs <= eng_mod.MAX_GRAPHS < engine.graphs_captured
    assert batch_sizes == len(sizes) and logits_bytes == min(eng_mod.SHARED_LOGITS_ROWS, engine.cache.n_slots) * vocab * 4
    # the first batch size's graph is long gone: it is captured again and agrees with eager steps
    s, se = engine.alloc_slot(), eager.alloc_slot()
    engine.step([StepEntry(s, feed[:200], [])]); eager.step([StepEntry(se, feed[:200], [])])
    before = engine.graphs_captured
    for j in range(4):
        a = engine.step([StepEntry(s, [feed[j]], [0])]).cpu().numpy()
        b = eager.step([StepEntry(se, [feed[j]], [0])]).cpu().numpy()
        assert np.array_equal(a, b)
    assert engine.graphs_captured == before + 1 and engine.decode_graph_stats()[0] <= eng_mod.MAX_GRAPHS
    engine.cache.check()


def test_generation_of_an_unequal_batch_whose_sequences_end_one_after_another(model_root):
    """The generation loop over one long prompt beside short ones, greedy, in bfloat16: the decode
    steps run one ahead of the host, as graphs, with the attention's grid dealt out by a list, and
    the caller ends the sequences at different counts, so that the batch shrinks step by step. Every
    token is at or near the top of what the plain implementation says for its place."""
    from herbert_rs_amd.sampling import SamplingParams
    folder = make_folder(model_root, "D", "bfloat16")
    vocab = CONFIGS["D"][0]["vocab_size"]
    prompts = [random_tokens(vocab, n, 800 + n) for n in (1500, 20, 300, 64, 5)]
    ends = [6, 25, 12, 30, 18]
    engine = hb.load(folder, dtype="bfloat16", cache_tokens=64 * 40)
    count = [0] * len(prompts)

    def on_token(i, tok):
        count[i] += 1
        return "enough" if count[i] >= ends[i] else None
    res = engine.generate(prompts, SamplingParams(temperature=0.0, max_tokens=40, ignore_eos=True, repeat_check=False),
                          on_token=on_token)
    assert [len(r.tokens) for r in res] == ends and engine.graphs_captured >= 4
    assert any(st.static.range_lists for st in engine._decode.values())           # the list was what ran
    for p, r in zip(prompts, res):
        ref = plain_logits(folder, p + r.tokens)
        for k, tok in enumerate(r.tokens):
            row = ref[len(p) + k - 1]
            assert float(row.max() - row[tok]) <= 0.05 * float(row.std()), (len(p), k)
    engine.cache.check()


def test_a_larger_batch_makes_a_larger_logits_buffer(model_root):
    """The decode steps' one logits buffer has 64 rows at first; a batch of 70 sequences makes one
    of 128 (every graph is dropped with the old one), and steps of 3, of 70 and of 3 again say
    what eager steps say."""
    folder = make_folder(model_root, "A", "bfloat16")
    vocab = CONFIGS["A"][0]["vocab_size"]
    engine = hb.Engine.from_folder(folder, dtype="bfloat16", max_tokens=64 * 140, max_slots=130, use_graphs=True)
    eager = hb.Engine.from_folder(folder, dtype="bfloat16", max_tokens=64 * 140, max_slots=130, use_graphs=False)
    feed = random_tokens(vocab, 400, 77)
    for B, rows in ((3, 64), (70, 128), (3, 128)):
        slots, slots_e = [engine.alloc_slot() for _ in range(B)], [eager.alloc_slot() for _ in range(B)]
        for eng, sl in ((engine, slots), (eager, slots_e)):
            eng.step([StepEntry(s, feed[i:i + 5 + i % 7], []) for i, s in enumerate(sl)])
        for j in range(4):
            toks = [feed[(11 * i + j) % len(feed)] for i in range(B)]
            a = engine.step([StepEntry(s, [t], [0]) for s, t in zip(slots, toks)]).cpu().numpy()
            b = eager.step([StepEntry(s, [t], [0]) for s, t in zip(slots_e, toks)]).cpu().numpy()
            assert a.shape == (B, vocab) and np.array_equal(a, b), (B, j)
        assert engine.decode_graph_stats()[2] == rows * vocab * 4
        for s in slots:
            engine.free_slot(s)
        for s in slots_e:
            eager.free_slot(s)
    # the first graph of 3 sequences went with the smaller buffer: 70 and 3 are kept, 3 was captured twice
    assert engine.decode_graph_stats()[:2] == (2, 2) and engine.graphs_captured == 3
    engine.cache.check()


def write_tokenizer(folder, vocab, renamed=None):
    """A tokenizer.json of whole words w0, w1, ... and the chat format's special tokens, written
    with the tokenizers package; the model's last ids are the specials. `renamed`: {id: word} for
    ids that are to be other words than w<id>."""
    from tokenizers import Tokenizer, decoders, models, pre_tokenizers
    specials = ["<|im_start|>", "<|im_end|>", "system", "user", "assistant"]
    words = {(renamed or {}).get(i, f"w{i}"): i for i in range(vocab - len(specials))}
    for i, t in enumerate(specials):
        words[t] = vocab - len(specials) + i
    tok = Tokenizer(models.WordLevel(words, unk_token="w0"))
    tok.pre_tokenizer = pre_tokenizers.WhitespaceSplit()
    tok.add_special_tokens(["<|im_start|>", "<|im_end|>"])
    tok.save(os.path.join(folder, "tokenizer.json"))
    return tok, words


def cli_folder(model_root, tmp_path, name="A"):
    src = make_folder(model_root, name, "float32")
    folder = str(tmp_path / f"{name}_text")
    os.makedirs(folder)
    os.link(os.path.join(src, "model.safetensors"), os.path.join(folder, "model.safetensors"))
    with open(os.path.join(src, "config.json")) as f:
        raw = json.load(f)
    raw["eos_token_id"] = 0                       # "w0": not among what this model says here
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(raw, f)
    return folder, raw


def run_cli(folder, *args, timeout=240):
    return subprocess.run([sys.executable, os.path.join(ROOT, "bin", "herbert-cli"), "--model", folder,
                           "--dtype", "float32", "--temperature", "0", "--no-repeat-check", *args],
                          capture_output=True, text=True, timeout=timeout)


def test_cli_with_a_tokenizer_chat_template_and_stop_strings(model_root, tmp_path):
    """With a tokenizer.json the prompt is text in the architecture's chat template
    (crates/cli/src/main.rs:281-294), the output is text, and --stop ends it where the decoded
    text first holds the string (main.rs:236-247,1328-1332,1360), the token that completes the
    string still printed."""
    folder, raw = cli_folder(model_root, tmp_path)
    tok, words = write_tokenizer(folder, raw["vocab_size"])
    prompt = "w5 w17 w3"
    ids = tok.encode("<|im_start|>system\nw9<|im_end|>\n<|im_start|>user\n" + prompt +
                     "<|im_end|>\n<|im_start|>assistant\n", add_special_tokens=False).ids
    assert ids[0] == words["<|im_start|>"] and words["w17"] in ids and len(ids) == 12
    cfg, w = plain_folder(folder)
    want = plain.greedy(cfg, w, ids, 13, stop_ids=(words["<|im_end|>"], 0))
    out = run_cli(folder, "--prompt", prompt, "--system", "w9", "--max-tokens", "12", "--verbose")
    assert out.returncode == 0, out.stderr
    text = tok.decode(want, skip_special_tokens=True)
    assert out.stdout.strip() == text.strip() and len(text.split()) >= 6
    # a stop string: the third and fourth words of what it says
    said = text.split()
    stop = " ".join(said[2:4])
    upto = next(n for n in range(1, len(said) + 1) if stop in " ".join(said[:n]))
    out = run_cli(folder, "--prompt", prompt, "--system", "w9", "--max-tokens", "12", "--verbose",
                  "--stop", stop, "--stop", "never said\\n")
    assert out.returncode == 0, out.stderr
    assert out.stdout.strip() == " ".join(said[:upto]) and upto <= 4
    assert "Stop reason:     stop_sequence" in out.stderr and f"Output tokens:   {upto}" in out.stderr


def test_cli_think_budget_system_file_and_prompt_in_pieces(model_root, tmp_path):
    """--think-budget caps a think block as the reference's sampler does
    (crates/core/src/sampler.rs:200-243): the tokenizer here calls an ordinary word that the model
    says once <think>, so the block opens by itself; after budget - 1 tokens the line break's id (the
    architecture's own, the tokenizer has none) is forced, then </think>, then the model goes on
    freely. --nothink is a budget of one. The system prompt comes from a file and the prompt goes
    through the engine in pieces of 5 tokens; neither changes a token."""
    from .plain.sampler import think_forced
    folder, raw = cli_folder(model_root, tmp_path, "C")      # (a model that says many different words)
    tok, words = write_tokenizer(folder, raw["vocab_size"])
    prompt = "w5 w17 w3"
    text = "<|im_start|>system\nw9<|im_end|>\n<|im_start|>user\n" + prompt + "<|im_end|>\n<|im_start|>assistant\n"
    ids = tok.encode(text, add_special_tokens=False).ids
    cfg, w = plain_folder(folder)
    free = plain.greedy(cfg, w, ids, 12)
    newline_id = 198
    # an ordinary word that the model says once becomes <think> (said again it would open a new block)
    at = next((j for j, t in enumerate(free[:6]) if t < raw["vocab_size"] - 5 and t not in ids and t != newline_id
               and free.count(t) == 1), None)
    assert at is not None, free
    open_id = free[at]
    close_id = next(i for i in range(20, 200) if i not in free and i not in ids and i != newline_id)
    tok, words = write_tokenizer(folder, raw["vocab_size"], {open_id: "<think>", close_id: "</think>"})
    assert tok.encode(text, add_special_tokens=False).ids == ids and tok.token_to_id("<think>") == open_id

    def capped(budget, n):
        out = []
        for _ in range(n):
            logits = plain.forward(cfg, w, ids + out)[-1]
            forced = think_forced(out, budget, open_id, close_id, newline_id)
            out.append(forced if forced is not None else plain.argmax(logits))
        return out

    system = tmp_path / "system.txt"
    system.write_text("w9")
    for flags, budget in ((["--think-budget", "3"], 3), (["--nothink"], 1)):
        n = at + budget + 4
        want = capped(budget, n)
        assert want[at] == open_id and want[at + budget] == newline_id and want[at + budget + 1] == close_id
        assert close_id not in capped(0, n)
        out = run_cli(folder, "--prompt", prompt, "--system-file", str(system), "--max-tokens", str(n - 1),
                      "--ignore-eos", "--prefill-chunk-size", "5", "--show-specials", *flags)
        assert out.returncode == 0, out.stderr
        assert out.stdout.strip() == tok.decode(want, skip_special_tokens=False).strip(), (out.stdout, want)
    # think tokens that the model's vocabulary does not hold are refused, not sampled
    write_tokenizer(folder, raw["vocab_size"])
    out = run_cli(folder, "--prompt", prompt, "--max-tokens", "4", "--nothink")
    assert out.returncode == 1 and "outside the model's vocabulary" in out.stderr


def test_cli_interrupt_ends_generation_cleanly(model_root, tmp_path):
    """SIGINT sets a flag that the loop looks at before its next decode step
    (crates/cli/src/main.rs:22-50,1242-1245): the process ends by itself with what it has."""
    folder = make_folder(model_root, "D", "float32")
    proc = subprocess.Popen([sys.executable, os.path.join(ROOT, "bin", "herbert-cli"), "--model", folder,
                             "--dtype", "float32", "--temperature", "0", "--no-repeat-check", "--ignore-eos",
                             "--prompt", "1,2,3", "--max-tokens", "2040", "--verbose"],
                            stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True)
    first = proc.stdout.read(1)                    # the first token is out: generation runs
    assert first.isdigit()
    proc.send_signal(signal.SIGINT)
    try:
        out, err = proc.communicate(timeout=120)
    finally:
        if proc.poll() is None:
            proc.kill()
    assert proc.returncode == 0, err
    tokens = (first + out).strip().split(",")
    assert "Interrupted" in err and "Stop reason:     interrupted" in err
    assert 1 <= len(tokens) < 2041 and all(t.isdigit() for t in tokens)


def test_cli_conversation_goes_on_in_its_slot(model_root, tmp_path):
    """Without a prompt the command line is a conversation (crates/cli/src/main.rs:718-757,
    crates/cli/src/chat.rs:601-1331): every turn goes on from what the cache holds. What the
    model says in a turn is what the plain implementation says after the whole conversation so
    far as one sequence: the earlier turns, each one's last token and end-of-turn token, the
    new message in the template. A stop string cuts the turns short, so that each ends on a
    token's value with the next step already run: that step is rolled back. /clear starts over
    and gives the first turn's answer again."""
    folder, raw = cli_folder(model_root, tmp_path, "C")      # (a model that says many different words)
    tok, words = write_tokenizer(folder, raw["vocab_size"])
    cfg, w = plain_folder(folder)
    im_end = words["<|im_end|>"]
    limit = 8

    def template(message, system=None):
        head = f"<|im_start|>system\n{system}<|im_end|>\n" if system else ""
        return tok.encode(head + "<|im_start|>user\n" + message + "<|im_end|>\n<|im_start|>assistant\n",
                          add_special_tokens=False).ids

    def reply(sequence, stop=None):
        said = plain.greedy(cfg, w, sequence, limit, stop_ids=(im_end, 0))
        if stop is not None:
            for n in range(1, len(said) + 1):
                if stop in tok.decode(said[:n], skip_special_tokens=True):
                    return said[:n]
        return said

    first = template("w5 w17 w3", "w9")
    free = reply(first)
    stop = tok.decode(free[2:3], skip_special_tokens=True).strip()     # the third word it says
    r1 = reply(first, stop)
    assert 1 <= len(r1) <= 3
    second = first + r1 + [im_end] + template("w40 w41")
    r2 = reply(second, stop)
    third = second + r2 + ([] if r2[-1] == im_end else [im_end]) + template("w7")
    r3 = reply(third, stop)
    lines = ["w5 w17 \\", "w3", "/stats", "w40 w41", "w7", "/clear", "w5 w17 w3", "/stats", "/quit"]
    out = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "herbert-cli"), "--model", folder, "--dtype", "float32",
                          "--temperature", "0", "--no-repeat-check", "--system", "w9", "--max-tokens", str(limit),
                          "--stop", stop, "--cache-tokens", "512"],
                         input="\n".join(lines) + "\n", capture_output=True, text=True, timeout=240)
    assert out.returncode == 0, out.stderr
    said = [l.strip() for l in out.stdout.split("\n") if l.strip()]
    want = [tok.decode(r, skip_special_tokens=True).strip() for r in (r1, r2, r3, r1)]
    assert said == want, (out.stdout, want)
    held = len(first) + len(r1) - 1
    assert f"KV cache tokens: {held}" in out.stderr and "[Conversation cleared]" in out.stderr
    assert out.stderr.count("Turns:") == 2 and "Turns:           4" in out.stderr
