"""The engine through its Python entry points: long decoding, greedy generation, slots used
again, the window's edge, errors of the step function, sampling on the GPU."""
import json
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

import herbert_rs_amd as hb
from herbert_rs_amd.engine import StepEntry
from herbert_rs_amd.errors import CacheError, RequestError

from .plain import model as plain
from .plain import sampler as plain_sampler
from .plain_cache import plain_folder, plain_logits
from .tiny import CONFIGS, make_folder, random_tokens

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


from .bounds import close


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["B", "C"])
def test_long_decoding_one_token_at_a_time(name, dtype, model_root):
    """A short prompt, then hundreds of single tokens: across page edges, beyond the window, up
    to the model's last position."""
    folder = make_folder(model_root, name, dtype)
    raw = CONFIGS[name][0]
    n = raw["max_position_embeddings"] if name == "B" else 330
    tokens = random_tokens(raw["vocab_size"], n, 5)
    engine = hb.load(folder, dtype=dtype, cache_tokens=n + 64)
    slot = engine.alloc_slot()
    ref = plain_logits(folder, tokens)
    got = [engine.step([StepEntry(slot, tokens[:3], [0, 1, 2])]).cpu().numpy()]
    for p in range(3, n):
        got.append(engine.step([StepEntry(slot, [tokens[p]], [0])]).cpu().numpy())
    got = np.concatenate(got)
    for p in range(n):
        ok, err = close(got[p], ref[p], dtype, name)
        assert ok, f"position {p}: err {err}"
    if name == "B":
        with pytest.raises(RequestError, match="max_position_embeddings"):
            engine.step([StepEntry(slot, [1], [0])])
    engine.free_slot(slot)
    engine.cache.check()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_chunks_of_a_prompt_and_slots_used_again(dtype, model_root):
    """A prompt fed in uneven pieces gives the logits of the whole; a slot that held another
    sequence gives the same logits as a fresh one."""
    folder = make_folder(model_root, "C", dtype)
    vocab = CONFIGS["C"][0]["vocab_size"]
    a, b = random_tokens(vocab, 150, 8), random_tokens(vocab, 90, 9)
    engine = hb.load(folder, dtype=dtype, cache_tokens=64 * 6)
    s = engine.alloc_slot()
    whole = engine.step([StepEntry(s, a, list(range(len(a))))]).cpu().numpy()
    engine.free_slot(s)
    s2 = engine.alloc_slot()
    assert s2 == s
    engine.step([StepEntry(s2, b, [])])                       # leaves other keys in the pages
    engine.free_slot(s2)
    s3 = engine.alloc_slot()
    pieces, at = [], 0
    for n in (1, 63, 1, 20, 65):
        pieces.append(engine.step([StepEntry(s3, a[at:at + n], list(range(n)))]).cpu().numpy())
        at += n
    pieces = np.concatenate(pieces)
    ref = plain_logits(folder, a)
    for p in range(len(a)):
        assert close(whole[p], ref[p], dtype, "C")[0] and close(pieces[p], ref[p], dtype, "C")[0], p
    if dtype == "float32":
        assert float(np.abs(pieces - whole).max()) <= 2e-5
    engine.free_slot(s3)
    engine.cache.check()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_prompts_with_heads_of_128(dtype, model_root, monkeypatch):
    """Heads of 128 and prompts of more than a thousand tokens: in bfloat16 the q/k/v projection
    then norms, rotates and writes the cache itself (for a product whose tiles fill the GPU; this
    small model's are let in by hand), and decoding does so inside its attention kernel. Whole, in
    a batch with a short prompt, in pieces, and decoded on: the plain logits."""
    from herbert_rs_amd.kernels import mfma
    monkeypatch.setattr(mfma, "QKV_FUSE_MIN_TILES", 16)
    fused = []
    real = mfma.gemm_qkv
    monkeypatch.setattr(mfma, "gemm_qkv", lambda *a, **k: (
        fused.append(mfma.qkv_tile_shape(a[0].shape[0], a[1].shape[0])), real(*a, **k))[1])
    folder = make_folder(model_root, "D", dtype)
    vocab = CONFIGS["D"][0]["vocab_size"]
    a, b = random_tokens(vocab, 1100, 30), random_tokens(vocab, 45, 31)
    ref_a, ref_b = plain_logits(folder, a), plain_logits(folder, b)
    at = [0, 1, 63, 64, 500, 1023, 1024, 1087, 1088, 1099]          # rows of the first and of the last tiles
    engine = hb.load(folder, dtype=dtype, cache_tokens=64 * 40)
    s = engine.alloc_slot()
    whole = engine.step([StepEntry(s, a[:1090], at[:-1])]).cpu().numpy()
    for row, p in enumerate(at[:-1]):
        assert close(whole[row], ref_a[p], dtype, "D")[0], p
    for p in range(1090, 1100):                                       # decoded on, one token a step
        got = engine.step([StepEntry(s, [a[p]], [0])]).cpu().numpy()[0]
        assert close(got, ref_a[p], dtype, "D")[0], p
    engine.free_slot(s)
    s1, s2 = engine.alloc_slot(), engine.alloc_slot()                 # two prompts of unequal length in one step
    both = engine.step([StepEntry(s1, b, [0, 44]), StepEntry(s2, a, [0, 1099])]).cpu().numpy()
    for row, (ref, p) in enumerate(((ref_b, 0), (ref_b, 44), (ref_a, 0), (ref_a, 1099))):
        assert close(both[row], ref[p], dtype, "D")[0], (row, p)
    engine.free_slot(s1)
    engine.free_slot(s2)
    s3 = engine.alloc_slot()                                          # pieces: short ones take the other kernels
    engine.step([StepEntry(s3, a[:70], [])])
    piece = engine.step([StepEntry(s3, a[70:], [1099 - 70])]).cpu().numpy()[0]
    assert close(piece, ref_a[1099], dtype, "D")[0]
    engine.free_slot(s3)
    # shorter prompts: the projection's smaller tiles (a head wide, 256 and 128 rows high)
    for n in (600, 250):
        s4 = engine.alloc_slot()
        rows = [p for p in (0, 127, 128, 255, 256) if p < n] + [n - 1]
        got = engine.step([StepEntry(s4, a[:n], rows)]).cpu().numpy()
        for row, p in enumerate(rows):
            assert close(got[row], ref_a[p], dtype, "D")[0], (n, p)
        engine.free_slot(s4)
    engine.cache.check()
    assert (len(fused) > 0) == (dtype == "bfloat16")
    if dtype == "bfloat16":
        assert set(fused) == {0, 1, 2}, fused           # every tile shape was taken by the host's own choice


ODD_SIZES = {
    # a vocabulary and a width that no kernel's block divides, seven heads on one kv head
    "odd_vocab": dict(vocab_size=323, hidden_size=72, intermediate_size=100, num_attention_heads=7,
                      num_key_value_heads=1, head_dim=16, eos_token_id=1),
    # widths in steps of 32 (the matrix-core products) with a vocabulary that is not one of 16
    "mfma_odd_vocab": dict(vocab_size=1001, hidden_size=160, intermediate_size=352, num_attention_heads=6,
                           num_key_value_heads=3, head_dim=64, eos_token_id=1),
    # head sizes in steps of 16 that the matrix-core attention does not take
    "head_80": dict(vocab_size=400, hidden_size=128, intermediate_size=192, num_attention_heads=4,
                    num_key_value_heads=2, head_dim=80, eos_token_id=1),
    "head_112": dict(vocab_size=272, hidden_size=96, intermediate_size=160, num_attention_heads=3,
                     num_key_value_heads=3, head_dim=112, eos_token_id=1),
    # the largest head the attention kernels take
    "head_512": dict(vocab_size=256, hidden_size=64, intermediate_size=96, num_attention_heads=2,
                     num_key_value_heads=1, head_dim=512, eos_token_id=1),
    # forty query heads to one kv head: more than the matrix-core attention shares a key among
    "group_40": dict(vocab_size=256, hidden_size=64, intermediate_size=96, num_attention_heads=40,
                     num_key_value_heads=1, head_dim=32, eos_token_id=1),
}


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", sorted(ODD_SIZES))
def test_sizes_that_fit_no_kernels_blocks(name, dtype, model_root):
    """Sizes that the configuration allows and that the fast kernels' blocks do not divide: the
    engine takes another kernel for them (never a wrong result): a prompt whole, a batch of
    unequal prompts, and tokens decoded on, against the plain logits."""
    folder = make_folder(model_root, "A", dtype, overrides=ODD_SIZES[name])
    vocab = ODD_SIZES[name]["vocab_size"]
    a, b = random_tokens(vocab, 100, 40), random_tokens(vocab, 13, 41)
    ref_a, ref_b = plain_logits(folder, a), plain_logits(folder, b)
    engine = hb.load(folder, dtype=dtype, cache_tokens=64 * 6)
    s1, s2 = engine.alloc_slot(), engine.alloc_slot()
    got = engine.step([StepEntry(s1, a[:90], [0, 63, 64, 89]), StepEntry(s2, b[:9], [0, 8])]).cpu().numpy()
    for row, (ref, p) in enumerate(((ref_a, 0), (ref_a, 63), (ref_a, 64), (ref_a, 89), (ref_b, 0), (ref_b, 8))):
        ok, err = close(got[row], ref[p], dtype, "odd")
        assert ok, f"prompt row {row} position {p}: err {err}"
    for k in range(10):
        entries = [StepEntry(s1, [a[90 + k]], [0])] + ([StepEntry(s2, [b[9 + k]], [0])] if k < 4 else [])
        got = engine.step(entries).cpu().numpy()
        ok, err = close(got[0], ref_a[90 + k], dtype, "odd")
        assert ok, f"decoded {90 + k}: err {err}"
        if k < 4:
            ok, err = close(got[1], ref_b[9 + k], dtype, "odd")
            assert ok, f"decoded {9 + k} of the short one: err {err}"
    engine.free_slot(s1)
    engine.free_slot(s2)
    engine.cache.check()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_head_too_large_is_refused(dtype, model_root):
    """Heads of more than 512 are beyond every attention kernel: a clear error, no result."""
    from herbert_rs_amd.errors import BackendError
    folder = make_folder(model_root, "A", dtype, overrides=dict(head_dim=528, num_attention_heads=2,
                                                                num_key_value_heads=1))
    with pytest.raises(BackendError, match="head"):
        engine = hb.load(folder, dtype=dtype, cache_tokens=128)
        slot = engine.alloc_slot()
        engine.step([StepEntry(slot, [1, 2, 3], [2])])


def test_a_batch_of_more_than_64_decodes_like_each_sequence_alone(model_root):
    """With more than 64 sequences a decode step is no longer a skinny product: the tiled kernels
    (and, in bfloat16, HIP graphs of them) take over. Every sequence must still get the logits
    it gets alone."""
    folder = make_folder(model_root, "D", "bfloat16")
    vocab = CONFIGS["D"][0]["vocab_size"]
    B = 80
    prompts = [random_tokens(vocab, 3 + (7 * i) % 40, 100 + i) for i in range(B)]
    nexts = [random_tokens(vocab, 4, 500 + i) for i in range(B)]
    engine = hb.load(folder, dtype="bfloat16", cache_tokens=64 * 2 * B)
    slots = [engine.alloc_slot() for _ in range(B)]
    engine.step([StepEntry(s, p, []) for s, p in zip(slots, prompts)])
    steps = [engine.step([StepEntry(s, [n[j]], [0]) for s, n in zip(slots, nexts)]).cpu().numpy() for j in range(4)]
    for s in slots:
        engine.free_slot(s)
    for i in (0, 1, 17, 40, 63, 64, 79):
        ref = plain_logits(folder, prompts[i] + nexts[i])
        for j in range(4):
            ok, err = close(steps[j][i], ref[len(prompts[i]) + j], "bfloat16", "D")
            assert ok, (i, j, err)
    engine.cache.check()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_heads_rotated_in_part(dtype, model_root):
    """partial_rotary_factor 0.5: the first half of a head is rotated, the rest is left as it is."""
    folder = make_folder(model_root, "B", dtype, overrides={"partial_rotary_factor": 0.5})
    vocab = CONFIGS["B"][0]["vocab_size"]
    tokens = random_tokens(vocab, 90, 44)
    ref = plain_logits(folder, tokens)
    full = plain_logits(make_folder(model_root, "B", dtype), tokens)
    assert float(np.abs(ref - full).max()) > 1e-2                     # the factor does matter
    engine = hb.load(folder, dtype=dtype, cache_tokens=128)
    s = engine.alloc_slot()
    got = engine.step([StepEntry(s, tokens[:70], list(range(70)))]).cpu().numpy()
    for p in range(70):
        assert close(got[p], ref[p], dtype, "B")[0], p
    for p in range(70, 90):
        assert close(engine.step([StepEntry(s, [tokens[p]], [0])]).cpu().numpy()[0], ref[p], dtype, "B")[0], p
    engine.free_slot(s)


def test_yarn_scaled_rotation_through_the_engine(model_root):
    over = {"rope_scaling": {"rope_type": "yarn", "factor": 4.0, "original_max_position_embeddings": 64}}
    raw, seed, std = CONFIGS["B"]
    folder = os.path.join(str(model_root), "B_yarn")
    if not os.path.exists(os.path.join(folder, "model.safetensors")):
        from herbert_rs_amd.weights import write_model_folder
        from herbert_rs_amd.engine.model import Model
        from .tiny import spec_of
        cfg, spec = spec_of(dict(raw, **over))
        write_model_folder(folder, dict(raw, **over), Model(spec).tensor_needs(), seed, dtype="float32", std=std, norm_std=0.1)
    tokens = random_tokens(raw["vocab_size"], 120, 45)
    ref = plain_logits(folder, tokens)
    assert float(np.abs(ref - plain_logits(make_folder(model_root, "B", "float32"), tokens)).max()) > 1e-2
    engine = hb.load(folder, dtype="float32", cache_tokens=128)
    s = engine.alloc_slot()
    got = engine.step([StepEntry(s, tokens, list(range(120)))]).cpu().numpy()
    assert float(np.abs(got - ref).max()) <= 1e-4
    engine.free_slot(s)


def test_window_edge_shows_in_the_logits(model_root):
    """Config C's first layer sees 70 keys. Changing the token just outside every later query's
    window must change nothing there; changing the one just inside must."""
    folder = make_folder(model_root, "C", "float32")
    raw = CONFIGS["C"][0]
    base = random_tokens(raw["vocab_size"], 120, 12)
    engine = hb.load(folder, dtype="float32", cache_tokens=256)

    def last_logits(tokens):
        s = engine.alloc_slot()
        out = engine.step([StepEntry(s, tokens, [len(tokens) - 1])]).cpu().numpy()[0]
        engine.free_slot(s)
        return out
    ref = last_logits(base)
    assert float(np.abs(ref - plain_logits(folder, base)[-1]).max()) <= 1e-4
    # the second layer sees everything, so any earlier token reaches the last logits; the check
    # is therefore made against the plain implementation on both sides of the edge
    for changed in (119 - 70, 119 - 69):
        other = list(base)
        other[changed] = (other[changed] + 1) % raw["vocab_size"]
        got = last_logits(other)
        assert float(np.abs(got - plain_logits(folder, other)[-1]).max()) <= 1e-4


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B"])
def test_greedy_generation_through_the_entry_point(name, dtype, model_root):
    folder = make_folder(model_root, name, dtype)
    raw, _, _ = CONFIGS[name]
    prompts = [random_tokens(raw["vocab_size"], n, 40 + n) for n in ((5, 11, 2) if name == "A" else (1, 17, 33, 9))]
    new = 8 if name == "A" else 12
    got = hb.generate(folder, prompts, temperature=0.0, max_tokens=new, ignore_eos=True,
                      no_repeat_check=True, dtype=dtype, max_batch=3)
    cfg, w = plain_folder(folder)
    for p, g in zip(prompts, got):
        assert len(g) == new
        if dtype == "float32":
            assert g == plain.greedy(cfg, w, p, new)
        else:
            seq = list(p)
            for tok in g:           # bfloat16 may swap near-equal logits; the choice must be near the top
                logits = plain.forward(cfg, w, seq)[-1]
                assert float(logits.max() - logits[tok]) <= 0.05 * float(logits.std())
                seq.append(tok)


def test_generation_stops_on_eos_and_other_sequences_go_on(model_root):
    folder = make_folder(model_root, "A", "float32")
    cfg, w = plain_folder(folder)
    prompts = [random_tokens(256, n, 60 + n) for n in (4, 9, 6)]
    want = [plain.greedy(cfg, w, p, 10) for p in prompts]
    eos = want[1][3]                                   # make the 4th token of request 1 the eos
    with open(os.path.join(folder, "config.json")) as f:
        raw = json.load(f)
    other = os.path.join(os.path.dirname(folder), "A_eos")
    os.makedirs(other, exist_ok=True)
    raw["eos_token_id"] = eos
    with open(os.path.join(other, "config.json"), "w") as f:
        json.dump(raw, f)
    if not os.path.exists(os.path.join(other, "model.safetensors")):
        os.link(os.path.join(folder, "model.safetensors"), os.path.join(other, "model.safetensors"))
    engine = hb.load(other, dtype="float32", cache_tokens=64 * 3)
    from herbert_rs_amd.sampling import SamplingParams
    res = engine.generate(prompts, SamplingParams(temperature=0.0, max_tokens=10, repeat_check=False))
    for r, wnt in zip(res, want):
        cut = wnt.index(eos) + 1 if eos in wnt else len(wnt)
        assert r.tokens == wnt[:cut]
        assert r.stop_reason == ("eos" if eos in wnt else "max_tokens")
    assert res[1].stop_reason == "eos" and len(res[1].tokens) <= 4
    engine.cache.check()
    assert engine.cache.slots.held_count == 0


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_decoding_ahead_of_the_host_gives_what_step_by_step_gives(model_root, dtype):
    """The generation loop puts every decode step on the stream before it has read the tokens of
    the one before (they go from the sampler to the next step on the GPU). Same tokens and stop
    reasons as with the host in between, greedy and sampled, with sequences that end on a token's
    value in the middle of a batch (so that a step has run ahead for them and the batch shrinks),
    through pages' edges; in float32 the greedy tokens are the plain implementation's."""
    from herbert_rs_amd.engine.generate import Generator
    from herbert_rs_amd.sampling import SamplingParams
    folder = make_folder(model_root, "C", dtype)
    cfg, w = plain_folder(folder)
    prompts = [random_tokens(320, n, 80 + n) for n in (60, 9, 130, 3)]
    engine = hb.load(folder, dtype=dtype, cache_tokens=64 * 12)
    free = Generator(engine, run_ahead=False).generate(
        prompts, SamplingParams(temperature=0.0, max_tokens=24, ignore_eos=True, repeat_check=False))
    if dtype == "float32":
        assert [r.tokens for r in free] == [plain.greedy(cfg, w, p, 24) for p in prompts]
    stop = free[1].tokens[7]                          # request 1 ends at its 8th token, if not before
    for params in (SamplingParams(temperature=0.0, max_tokens=24, ignore_eos=True, repeat_check=False, stop_ids=(stop,)),
                   SamplingParams(temperature=0.9, top_k=12, top_p=0.95, seed=4, max_tokens=30, repeat_check=False),
                   SamplingParams(temperature=1.1, top_k=0, top_p=1.0, seed=9, max_tokens=17, repeat_check=False)):
        a = Generator(engine, run_ahead=False)
        b = Generator(engine, run_ahead=True)
        want = a.generate(prompts, params)
        got = b.generate(prompts, params)
        assert [(r.tokens, r.stop_reason) for r in got] == [(r.tokens, r.stop_reason) for r in want]
        assert b.stats.decode_steps >= a.stats.decode_steps
        engine.cache.check()
        assert engine.cache.slots.held_count == 0
    # the step function itself: tokens from the device give the logits that tokens from the host give
    s1, s2 = engine.alloc_slot(), engine.alloc_slot()
    engine.step([StepEntry(s1, prompts[0], []), StepEntry(s2, prompts[1], [])])
    host = engine.step([StepEntry(s1, [17], [0]), StepEntry(s2, [200], [0])]).clone()
    engine.truncate(s1, len(prompts[0]))
    engine.truncate(s2, len(prompts[1]))
    dev = torch.tensor([17, 200], dtype=torch.int32, device="cuda")
    fed = engine.step([StepEntry(s1, [0], [0]), StepEntry(s2, [0], [0])], tokens_on_device=dev)
    assert torch.equal(fed, host)
    with pytest.raises(RequestError, match="tokens_on_device"):
        engine.step([StepEntry(s1, [1, 2], [0])], tokens_on_device=dev[:1])
    # an id from the device that the vocabulary does not hold (the host cannot check it) reads nothing:
    # its row comes out NaN, the other sequence's row is what it would have been
    engine.truncate(s1, len(prompts[0]))
    engine.truncate(s2, len(prompts[1]))
    bad = torch.tensor([17, 1 << 20], dtype=torch.int32, device="cuda")
    fed = engine.step([StepEntry(s1, [0], [0]), StepEntry(s2, [0], [0])], tokens_on_device=bad)
    assert torch.equal(fed[0], host[0]) and bool(torch.isnan(fed[1]).all())
    engine.free_slot(s1)
    engine.free_slot(s2)
    # and without captured graphs (the step's metadata is then packed afresh every time)
    plain_steps = hb.Engine.from_folder(folder, dtype=dtype, max_tokens=64 * 12, use_graphs=False)
    got = Generator(plain_steps, run_ahead=True).generate(prompts, params)
    assert [(r.tokens, r.stop_reason) for r in got] == [(r.tokens, r.stop_reason) for r in want]


def test_get_tensor_gives_the_weights_as_stored(model_root):
    from safetensors.torch import load_file
    from herbert_rs_amd.errors import ModelLoadError
    folder = make_folder(model_root, "B", "bfloat16")
    stored = load_file(os.path.join(folder, "model.safetensors"))
    engine = hb.load(folder, dtype="bfloat16", cache_tokens=128)
    for name in ("model.layers.1.self_attn.q_proj.weight", "model.layers.2.mlp.gate_proj.weight", "lm_head.weight"):
        assert torch.equal(engine.get_tensor(name), stored[name])
    with pytest.raises(ModelLoadError, match="no tensor"):
        engine.get_tensor("model.layers.7.mlp.gate_proj.weight")
    from herbert_rs_amd.engine import Engine
    from herbert_rs_amd.config import load_config
    _, config = load_config(folder)
    seeded = Engine.from_config(config, seed=5, dtype="bfloat16", max_tokens=128)
    again = Engine.from_config(config, seed=5, dtype="bfloat16", max_tokens=128)
    t = seeded.get_tensor("model.layers.0.mlp.down_proj.weight")
    assert t.shape == (96, 224) and torch.equal(t, again.get_tensor("model.layers.0.mlp.down_proj.weight"))


def test_step_errors(model_root):
    folder = make_folder(model_root, "A", "float32")
    engine = hb.load(folder, dtype="float32", cache_tokens=128)
    s = engine.alloc_slot()
    with pytest.raises(RequestError, match="out of range"):
        engine.step([StepEntry(s, [256], [0])])
    with pytest.raises(RequestError, match="no tokens"):
        engine.step([StepEntry(s, [], [])])
    with pytest.raises(RequestError, match="twice"):
        engine.step([StepEntry(s, [1], [0]), StepEntry(s, [2], [0])])
    with pytest.raises(RequestError, match="outside"):
        engine.step([StepEntry(s, [1, 2], [2])])
    with pytest.raises(RequestError, match="max_position_embeddings"):
        engine.step([StepEntry(s, [1] * 129, [0])])
    with pytest.raises(CacheError):
        engine.step([StepEntry(5, [1], [0])])                 # a slot that is not held
    assert engine.step([StepEntry(s, [1, 2, 3], [])]) is None
    assert engine.cache.length(s) == 3
    engine.free_slot(s)
    engine.cache.check()


def test_cli_generates_token_ids(model_root):
    """--max-tokens counts the decode steps after the prompt's own token, as the reference's
    single shot does (crates/cli/src/main.rs:1040,1241): 6 gives 7 tokens."""
    folder = make_folder(model_root, "A", "float32")
    cfg, w = plain_folder(folder)
    out = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "herbert-cli"), "--model", folder,
                          "--prompt", "5,17,3", "--temperature", "0", "--max-tokens", "6", "--dtype",
                          "float32", "--ignore-eos", "--no-repeat-check", "--verbose"],
                         capture_output=True, text=True, timeout=240)
    assert out.returncode == 0, out.stderr
    assert [int(t) for t in out.stdout.strip().split(",")] == plain.greedy(cfg, w, [5, 17, 3], 7)
    assert "Prefill:" in out.stderr and "Decode:" in out.stderr and "Output tokens:   7" in out.stderr


# ---- sampling kernels against the plain sampler
@pytest.mark.parametrize("V", [5000, 70001])
def test_argmax_kernel_takes_the_first_of_equals(V):
    from herbert_rs_amd.kernels import ops
    logits = torch.randn(5, V)
    logits[0, 77] = logits[0, 4000] = 50.0
    logits[1, V - 1] = 60.0
    logits[2, 0] = 60.0
    logits[3] = -float("inf")
    out = torch.empty(5, dtype=torch.int32, device="cuda")
    ops.argmax(logits.cuda(), out)
    assert out.tolist() == [plain_sampler.argmax(r.numpy()) for r in logits]
    assert out.tolist()[:4] == [77, V - 1, 0, 0]
    # a row that holds NaN and nothing above -inf (what a token id out of range leaves of a step)
    # gives -1, which the generation loop reports; NaN beside finite values is passed over
    logits[3, V // 2] = float("nan")
    logits[4] = float("nan")
    logits[0, 5] = float("nan")
    ops.argmax(logits.cuda(), out)
    assert out.tolist() == [77, V - 1, 0, -1, -1]


@pytest.mark.parametrize("V", [1500, 10000])
@pytest.mark.parametrize("top_k,top_p", [(20, 1.0), (40, 0.9), (1, 1.0), (5, 0.3), (0, 1.0), (0, 0.8),
                                         (2000, 0.95), (300, 1.0)])
def test_sampler_matches_the_plain_sampler(top_k, top_p, V):
    """Same seed, same logits: the same token as the step-by-step host formulation, draw after
    draw; where the draw falls within rounding of a boundary either neighbour is right."""
    from herbert_rs_amd.kernels import ops
    from herbert_rs_amd.sampling import xorshift
    R, temperature = 6, 0.7
    g = torch.Generator().manual_seed(top_k + 3)
    logits = torch.randn(R, V, generator=g) * 2.0
    logits[1, 10] = logits[1, 900] = logits[1].max() + 0.5          # equal values at the top
    dev_logits = logits.cuda()
    seeds = [xorshift.sequence_seed(7, i) for i in range(R)]
    states = torch.tensor([s - (1 << 64) if s >= (1 << 63) else s for s in seeds], dtype=torch.int64,
                          device="cuda")
    index = torch.arange(R, dtype=torch.int32, device="cuda")
    p2 = 2048 if V <= 2048 else 16384
    scratch = (torch.empty(R, p2, dtype=torch.int32, device="cuda"),
               torch.empty(R, p2, dtype=torch.int32, device="cuda"))
    rngs = [plain_sampler.XorShift64(s) for s in seeds]
    out = torch.empty(R, dtype=torch.int32, device="cuda")
    for draw in range(12):
        ops.sample(dev_logits, temperature, top_k, top_p, states, index, out, scratch)
        got = out.tolist()
        for r in range(R):
            work = plain_sampler.candidates(logits[r].numpy(), temperature, top_k, top_p)
            u = rngs[r].next_f32()
            want = plain_sampler.pick(work, u)
            if got[r] != want:
                cum, near = np.float32(0), False
                for idx, p in work:
                    cum = np.float32(cum + p)
                    if abs(float(cum) - float(u)) < 1e-5:
                        near = True
                assert near and got[r] in [i for i, _ in work], (draw, r, got[r], want)
    assert [int(s) & ((1 << 64) - 1) for s in states.tolist()] == [r.state for r in rngs]


@pytest.mark.parametrize("V", [1500, 20000, 151936])
def test_top_p_without_top_k_looks_among_the_largest_first(V):
    """Top-p without top-k through the Sampler: a steep row is decided among its 1024 largest
    logits, a flat row and a row whose 1024th largest is one of 1990 equal ones are not (they get
    -1 from the quick kernel) and go the general way; all three give the plain sampler's tokens,
    draw after draw, and every generator advances once a draw."""
    from herbert_rs_amd.kernels import ops
    from herbert_rs_amd.sampling import SamplingParams, xorshift
    from herbert_rs_amd.sampling.sampler import Sampler
    temperature, top_p = 0.8, 0.85
    g = torch.Generator().manual_seed(V)
    steep = torch.randn(V, generator=g) * 6.0
    flat = torch.randn(V, generator=g) * 0.2
    level = torch.randn(V, generator=g) * 0.5 - 8.0
    # (1990 or V - 10 equal ones: top_p of them ends well inside a probability, not at its edge)
    level[torch.randperm(V, generator=g)[:min(1990, V - 10)]] = 3.0
    steep_tail = torch.randn(V, generator=g) * 5.0
    logits = torch.stack([steep, flat, level, steep_tail])
    R = logits.shape[0]
    dev_logits = logits.cuda()
    params = SamplingParams(temperature=temperature, top_k=0, top_p=top_p, max_tokens=4, seed=21)
    sampler = Sampler(params, R, V, torch.device("cuda"))
    rngs = [plain_sampler.XorShift64(xorshift.sequence_seed(21, i)) for i in range(R)]
    works = [plain_sampler.candidates(logits[r].numpy(), temperature, 0, top_p) for r in range(R)]
    assert len(works[0]) < 1024 < len(works[1])

    # which rows the quick kernel decides (on copies of the states: a row it leaves keeps its state)
    states = sampler.states.clone()
    out = torch.empty(R, dtype=torch.int32, device="cuda")
    ops.sample_nucleus(dev_logits, temperature, top_p, states, torch.arange(R, dtype=torch.int32, device="cuda"),
                       out, ops.nucleus_buffers(R, V, "cuda"))
    quick = [t >= 0 for t in out.tolist()]
    assert quick[:3] == [True, False, False]
    kept = [a == b for a, b in zip(states.tolist(), sampler.states.tolist())]
    assert kept == [not q for q in quick]

    for draw in range(10):
        got = sampler.choose(dev_logits, list(range(R)))
        for r in range(R):
            u = rngs[r].next_f32()
            want = plain_sampler.pick(works[r], u)
            if got[r] != want:
                cum, near = np.float32(0), False
                for idx, p in works[r]:
                    cum = np.float32(cum + p)
                    if abs(float(cum) - float(u)) < 1e-5:
                        near = True
                assert near and got[r] in [i for i, _ in works[r]], (draw, r, got[r], want)
    assert [int(s) & ((1 << 64) - 1) for s in sampler.states.tolist()] == [r.state for r in rngs]


@pytest.mark.parametrize("V", [8193, 20000, 151936])
def test_temperature_sampling_over_whole_long_rows(V):
    """No top-k, no top-p on rows of more than 8192 logits through the Sampler: the chunks of a row
    are added up side by side and the draw is looked for in the chunk it falls into; the plain
    sampler's tokens, draw after draw (either neighbour where the draw lies within rounding of a
    boundary), and the generators in step."""
    from herbert_rs_amd.sampling import SamplingParams, xorshift
    from herbert_rs_amd.sampling.sampler import Sampler
    temperature = 0.9
    g = torch.Generator().manual_seed(V + 1)
    logits = torch.stack([torch.randn(V, generator=g) * 3.0, torch.randn(V, generator=g) * 0.5,
                          torch.randn(V, generator=g) * 8.0, torch.randn(V, generator=g)])
    logits[3, 5000:] = -float("inf")                   # whole chunks without a finite logit
    R = logits.shape[0]
    dev_logits = logits.cuda()
    sampler = Sampler(SamplingParams(temperature=temperature, top_k=0, top_p=1.0, max_tokens=4, seed=5), R, V,
                      torch.device("cuda"))
    rngs = [plain_sampler.XorShift64(xorshift.sequence_seed(5, i)) for i in range(R)]
    works = [plain_sampler.candidates(logits[r].numpy(), temperature, 0, 1.0) for r in range(R)]
    # the same probabilities summed in float64: where the exact running sum passes a draw
    exact = [np.cumsum(np.array([p for _, p in w], dtype=np.float64)) for w in works]
    for draw in range(12):
        got = sampler.choose(dev_logits, list(range(R)))
        for r in range(R):
            u = rngs[r].next_f32()
            want = plain_sampler.pick(works[r], u)
            if got[r] != want:
                # A running sum of V float32 terms drifts by about sqrt(V) half-ulps, the plain sampler's
                # single one and the kernel's chunk by chunk differently, and so do their denominators:
                # among tokens of negligible probability the draw then falls on another one. What must
                # hold is that the token's stretch of the exact running sum lies within that drift of
                # the draw (a wrong chunk or an edge missed would be off by a chunk's share, per cents).
                drift = 8.0 * np.sqrt(V) * 2.0 ** -24
                g_ = got[r]
                assert exact[r][g_] >= u - drift and (g_ == 0 or exact[r][g_ - 1] <= u + drift), \
                    (draw, r, g_, want, float(exact[r][g_]), float(u))
    assert [int(s) & ((1 << 64) - 1) for s in sampler.states.tolist()] == [r.state for r in rngs]


@pytest.mark.parametrize("temperature", [0.0, 0.8])
def test_sampler_caps_a_think_block(temperature):
    """The Sampler with a think budget of 3: sequence 0 opens a block (its logits say so), then
    wants token 11 for ever: it gets 11, 11, the line break, the closing token, then 11 again;
    sequence 1 never opens one and is left alone. A forced row keeps one finite logit, and a
    draw is taken for it as for any row (crates/core/src/sampler.rs:72-145 runs on the forced
    logits), so the generators stay in step with the plain ones."""
    from herbert_rs_amd.sampling import SamplingParams, ThinkTokens, xorshift
    from herbert_rs_amd.sampling.sampler import Sampler
    V, ids = 3000, ThinkTokens(open_id=5, close_id=6, newline_id=7)
    params = SamplingParams(temperature=temperature, top_k=4, top_p=0.9, max_tokens=9, seed=3, think_budget=3,
                            think_tokens=ids)
    sampler = Sampler(params, 2, V, torch.device("cuda"))

    def logits_for(a, b):
        rows = torch.full((2, V), -4.0)
        rows[0, a] = rows[1, b] = 30.0
        return rows.cuda()

    got = []
    for step in range(7):
        logits = logits_for(5 if step == 0 else 11, 12)
        got.append(sampler.choose(logits, [0, 1]))
        if step in (3, 4):
            row = logits[0].cpu()
            assert torch.isfinite(row).sum() == 1 and torch.isfinite(row[7 if step == 3 else 6])
            assert torch.isfinite(logits[1]).all()
    assert [g[0] for g in got] == [5, 11, 11, 7, 6, 11, 11]
    assert [g[1] for g in got] == [12] * 7
    if temperature > 0:
        rngs = [plain_sampler.XorShift64(xorshift.sequence_seed(3, i)) for i in range(2)]
        for r in rngs:
            for _ in range(7):
                r.next_f32()
        assert [int(s) & ((1 << 64) - 1) for s in sampler.states.tolist()] == [r.state for r in rngs]


def test_sampler_draw_and_top_p_edge_on_exact_probabilities():
    """Equal logits give probabilities that are exact in float32 whatever the exponential's
    rounding (exp(0) = 1), so two rules show without a tolerance. (1) The draw is the upper bits
    of the new state over 2^24 (crates/core/src/sampler.rs:58-62): over 4096 equal logits the
    token is the state's upper 12 bits. (2) The top-p prefix ends where the running sum is
    >= top_p (sampler.rs:117-121): four equal logits and top_p 0.5 leave the first two tokens;
    with a strict comparison a third would be drawn about every third time."""
    from herbert_rs_amd.kernels import ops
    from herbert_rs_amd.sampling import xorshift
    seeds = [(1 << 63) + (1 << 36) + (1 << 33), 7, 0xDEADBEEF, 123456789123456789]
    R = len(seeds)

    def run(V, top_p, draws):
        logits = torch.full((R, V), 1.25, device="cuda")
        states = torch.tensor([s - (1 << 64) if s >= (1 << 63) else s for s in seeds], dtype=torch.int64,
                              device="cuda")
        index = torch.arange(R, dtype=torch.int32, device="cuda")
        p2 = 1
        while p2 < V:
            p2 <<= 1
        scratch = (torch.empty(R, p2, dtype=torch.int32, device="cuda"),
                   torch.empty(R, p2, dtype=torch.int32, device="cuda"))
        out = torch.empty(R, dtype=torch.int32, device="cuda")
        got = []
        for _ in range(draws):
            ops.sample(logits, 1.0, 0, top_p, states, index, out, scratch)
            got.append(out.tolist())
        return got

    got = run(4096, 1.0, 8)
    host = list(seeds)
    for d in range(8):
        host = [xorshift.step(s) for s in host]
        assert got[d] == [s >> 52 for s in host], d
    assert got[0][0] == 0x082                       # 0x08260C9224000000 >> 52, worked out by hand in test_plain
    got = run(4, 0.5, 40)
    seen = {t for row in got for t in row}
    assert seen == {0, 1}
    host = list(seeds)
    for d in range(40):                              # renormalised to a half each: the draw's top bit decides
        host = [xorshift.step(s) for s in host]
        assert got[d] == [s >> 63 for s in host], d


@pytest.mark.parametrize("sift", [False, True])
@pytest.mark.parametrize("V,levels,top_k", [(3000, 3, 40), (5000, 2, 1000), (151936, 40, 64), (2000, 1, 7),
                                            (17000, 5, 1000), (20000, 1000, 300), (151936, 100000, 1024)])
def test_sampler_with_many_equal_logits(V, levels, top_k, sift):
    """Logits that take few values: the k-th largest is then one of hundreds or thousands of equal
    ones (more than the kernel lists at once when V / levels exceeds 1024), and those with the
    lowest indices belong to the candidates. Same tokens as the host formulation, also when a
    block for every 8192 logits sifts the row first (17000: the last chunk is shorter than top_k)."""
    from herbert_rs_amd.kernels import ops
    from herbert_rs_amd.sampling import xorshift
    R, temperature, top_p = 3, 0.9, 1.0
    g = torch.Generator().manual_seed(V + top_k)
    logits = torch.randint(0, levels, (R, V), generator=g).float() * 0.5
    dev_logits = logits.cuda()
    seeds = [xorshift.sequence_seed(11, i) for i in range(R)]
    states = torch.tensor([s - (1 << 64) if s >= (1 << 63) else s for s in seeds], dtype=torch.int64, device="cuda")
    index = torch.arange(R, dtype=torch.int32, device="cuda")
    rngs = [plain_sampler.XorShift64(s) for s in seeds]
    out = torch.empty(R, dtype=torch.int32, device="cuda")
    works = [plain_sampler.candidates(logits[r].numpy(), temperature, top_k, top_p) for r in range(R)]
    for r in range(R):                 # the candidates are the top_k first indices of the highest level(s)
        assert len(works[r]) == top_k
    sifted = None
    if sift:
        need = R * -(-V // ops.SAMPLE_CHUNK) * top_k
        sifted = (torch.full((need,), -1, dtype=torch.int32, device="cuda"),
                  torch.full((need,), -1, dtype=torch.int32, device="cuda"))
    for draw in range(10):
        ops.sample(dev_logits, temperature, top_k, top_p, states, index, out, None, sifted)
        got = out.tolist()
        for r in range(R):
            u = rngs[r].next_f32()
            want = plain_sampler.pick(works[r], u)
            if got[r] != want:
                cum, near = np.float32(0), False
                for _, p in works[r]:
                    cum = np.float32(cum + p)
                    if abs(float(cum) - float(u)) < 1e-5:
                        near = True
                assert near and got[r] in [i for i, _ in works[r]], (draw, r, got[r], want)


def test_sampling_through_generate_is_reproducible(model_root):
    folder = make_folder(model_root, "B", "float32")
    prompts = [random_tokens(384, n, 70 + n) for n in (1, 17, 33, 9)]
    kw = dict(temperature=0.7, top_k=20, top_p=1.0, max_tokens=12, ignore_eos=True, no_repeat_check=True,
              dtype="float32", seed=7)
    a = hb.generate(folder, prompts, **kw)
    b = hb.generate(folder, prompts, **kw)
    c = hb.generate(folder, prompts, **dict(kw, seed=8))
    assert a == b and a != c and all(len(t) == 12 for t in a)
    # every request's tokens are those of the reference's sampler on the plain model's logits, each
    # request with the stream of its own seed (the first with the seed itself): every token of all
    # four; another token only where the draw lies within rounding of a boundary between two
    # candidates, and the comparison then goes on from the engine's token
    from herbert_rs_amd.sampling import xorshift
    cfg, w = plain_folder(folder)
    excused = 0
    for i, (prompt, tokens) in enumerate(zip(prompts, a)):
        rng = plain_sampler.XorShift64(xorshift.sequence_seed(7, i))
        seq = list(prompt)
        for n, tok in enumerate(tokens):
            logits = plain.forward(cfg, w, seq)[-1].numpy()
            work = plain_sampler.candidates(logits, 0.7, 20, 1.0)
            u = rng.next_f32()
            want = plain_sampler.pick(work, u)
            if tok != want:
                cum, near = np.float32(0), False
                for _, p in work:
                    cum = np.float32(cum + p)
                    near = near or abs(float(cum) - float(u)) < 1e-5
                assert near and tok in [j for j, _ in work], (i, n, tok, want)
                excused += 1
            seq.append(tok)
    assert excused <= 2


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_seed_gives_the_same_weights_on_the_gpu_and_in_a_folder(dtype, tmp_path):
    """Engine.from_config draws its weights on the GPU, write_random_model on the host: the same
    seed gives the same bits, so what the benchmark times can be written out and compared with the
    plain implementation; and the two engines give the same logits."""
    from herbert_rs_amd.config.registry import resolve_architecture
    from .tiny import TINY_B
    arch = resolve_architecture(TINY_B)
    cfg = arch.config_class.from_dict(TINY_B)
    drawn = hb.Engine.from_config(cfg, seed=11, dtype=dtype, std=0.05, norm_std=0.1, max_tokens=128)
    folder = hb.write_random_model(str(tmp_path / "m"), TINY_B, seed=11, dtype=dtype, std=0.05, norm_std=0.1)
    read = hb.load(folder, dtype=dtype, cache_tokens=128)
    from safetensors import safe_open
    with safe_open(os.path.join(folder, "model.safetensors"), framework="pt") as f:
        names = list(f.keys())
        assert len(names) == 3 * 11 + 3
        for name in names:
            stored = f.get_tensor(name)
            again = drawn.get_tensor(name)
            assert stored.dtype == again.dtype and torch.equal(stored, again), name
    tokens = random_tokens(384, 40, 12)
    a = drawn.step([StepEntry(drawn.alloc_slot(), tokens, list(range(40)))]).cpu()
    b = read.step([StepEntry(read.alloc_slot(), tokens, list(range(40)))]).cpu()
    assert torch.equal(a, b)
    ref = plain_logits(folder, tokens)
    assert close(a[39].numpy(), ref[39], dtype, "B")[0]


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_padding_rows_of_a_decode_step_change_nothing(dtype, model_root):
    """Decode steps run at a ladder of batch sizes (5 sequences as 6, 7 as 8, 9 as 10, 17 as 20), the
    rows left over being padding in a slot and a page of their own. Every sequence's logits are
    what it gets alone (in float32 bit for bit: those kernels sum every output the same way whatever
    the batch), through eager steps, recordings and replays; the pages of the sequences hold what
    they hold without the padding; the padding's slot and page are nobody's."""
    from herbert_rs_amd.engine.batch import decode_batch_bucket
    name = "D"
    folder = make_folder(model_root, name, dtype)
    vocab = CONFIGS[name][0]["vocab_size"]
    assert [decode_batch_bucket(n) for n in (1, 2, 3, 4, 5, 7, 9, 16, 17, 33, 64, 65)] == \
        [1, 2, 3, 4, 6, 8, 10, 16, 20, 40, 64, 72]
    n_seqs, steps = 17, 6
    seqs = [random_tokens(vocab, 20 + 9 * i + steps, 400 + i) for i in range(n_seqs)]
    heads = [len(t) - steps for t in seqs]
    alone_engine = hb.load(folder, dtype=dtype, cache_tokens=64 * 8)
    alone = []
    for t, h in zip(seqs, heads):
        slot = alone_engine.alloc_slot()
        alone_engine.step([StepEntry(slot, t[:h], [])])
        alone.append(torch.stack([alone_engine.step([StepEntry(slot, [t[h + j]], [0])])[0] for j in range(steps)]).cpu())
        alone_engine.free_slot(slot)
    engine = hb.load(folder, dtype=dtype, cache_tokens=64 * 4 * n_seqs)
    pad_slot = engine.cache.pad_slot
    for n in (5, 7, 9, 17):
        slots = [engine.alloc_slot() for _ in range(n)]
        assert pad_slot not in slots
        engine.step([StepEntry(s, t[:h], []) for s, t, h in zip(slots, seqs, heads)])
        for j in range(steps):
            got = engine.step([StepEntry(s, [t[h + j]], [0]) for s, t, h in zip(slots, seqs, heads)]).cpu()
            assert got.shape == (n, vocab)
            for i in range(n):
                if dtype == "float32":
                    assert torch.equal(got[i], alone[i][j]), (n, j, i)
                else:
                    assert close(got[i].numpy(), alone[i][j].numpy(), dtype, name, "padded step")[0], (n, j, i)
        for s in slots:
            engine.free_slot(s)
        engine.cache.check()
    assert sorted(engine._decode) == [6, 8, 10, 20] and engine.graphs_captured >= 4
    for g in engine.cache.kv_groups.values():
        assert g.pages.held_count == 0 and int(g.table[pad_slot].min()) == g.pool.shape[2] - 1


def test_a_decode_steps_logits_are_the_callers_own(model_root):
    """What `step` returns for a decode step is a copy of the caller's own: the next decode step does
    not change it. Asked for the rows themselves (`keep_logits=False`, as the generation loop asks),
    the caller gets a view of the engine's buffer, which the next decode step writes again."""
    folder = make_folder(model_root, "B", "float32")
    tokens = random_tokens(384, 30, 61)
    engine = hb.load(folder, dtype="float32", cache_tokens=64 * 2)
    slot = engine.alloc_slot()
    engine.step([StepEntry(slot, tokens[:20], [])])
    own = engine.step([StepEntry(slot, [tokens[20]], [0])])
    kept = own.clone()
    view = engine.step([StepEntry(slot, [tokens[21]], [0])], keep_logits=False)
    seen = view.clone()
    assert torch.equal(own, kept) and not torch.equal(own, seen)
    nxt = engine.step([StepEntry(slot, [tokens[22]], [0])])
    assert torch.equal(own, kept) and torch.equal(view, nxt) and not torch.equal(view, seen)
    assert own.data_ptr() != view.data_ptr() and nxt.data_ptr() != view.data_ptr()
    ref = plain_logits(folder, tokens[:23])
    for got, p in ((own, 20), (seen, 21), (nxt, 22)):
        assert close(got[0].cpu().numpy(), ref[p], "float32", "B")[0], p


def test_two_engines_on_two_streams_share_no_scratch(model_root):
    """Each engine's kernels have scratch of their own (the partial results of the decode
    attention's ranges, the K slices of products): two engines of one process, stepped in turn on
    two streams without waiting for each other, give bit for bit what each gives alone."""
    folder = make_folder(model_root, "D", "bfloat16")
    seqs = [random_tokens(512, 700, 300 + i) for i in range(2)]

    def decode(engine, tokens, stream, out):
        with torch.cuda.stream(stream):
            slot = engine.alloc_slot()
            engine.step([StepEntry(slot, tokens[:640], [])])
        for p in range(640, 700):
            yield
            with torch.cuda.stream(stream):
                out.append(engine.step([StepEntry(slot, [tokens[p]], [0])]).clone())

    alone = []
    for t in seqs:
        engine = hb.load(folder, dtype="bfloat16", cache_tokens=64 * 12)
        got = []
        for _ in decode(engine, t, torch.cuda.current_stream(), got):
            pass
        torch.cuda.synchronize()
        alone.append(torch.stack(got).cpu())
    engines = [hb.load(folder, dtype="bfloat16", cache_tokens=64 * 12) for _ in seqs]
    assert engines[0].rt.scratch is not engines[1].rt.scratch
    streams = [torch.cuda.Stream() for _ in seqs]
    outs = [[], []]
    runs = [decode(e, t, s, o) for e, t, s, o in zip(engines, seqs, streams, outs)]
    live = list(runs)
    while live:                                  # a step of one, a step of the other, nobody waits
        for r in list(live):
            try:
                next(r)
            except StopIteration:
                live.remove(r)
    torch.cuda.synchronize()
    for e in engines:
        assert e.rt.scratch.partials, "the decode attention of heads of 128 keeps partial results"
    assert engines[0].rt.scratch.partials[-1][0].data_ptr() != engines[1].rt.scratch.partials[-1][0].data_ptr()
    for i in range(2):
        assert torch.equal(torch.stack(outs[i]).cpu(), alone[i]), i


def test_a_capture_that_fails_leaves_the_shape_to_start_over(model_root):
    """A forward pass that raises while a decode step is captured: the error reaches the caller,
    the cache is as before, and the shape's next step runs eagerly again instead of going straight
    into another capture; the step after that is captured, and replays give the eager logits."""
    folder = make_folder(model_root, "B", "float32")
    tokens = random_tokens(384, 40, 77)
    engine = hb.Engine.from_folder(folder, dtype="float32", max_tokens=64 * 4)
    plain_engine = hb.Engine.from_folder(folder, dtype="float32", max_tokens=64 * 4, use_graphs=False)
    slot, slot0 = engine.alloc_slot(), plain_engine.alloc_slot()
    engine.step([StepEntry(slot, tokens[:10], [])])
    plain_engine.step([StepEntry(slot0, tokens[:10], [])])
    real = engine.model.forward
    state = {"failed": 0}

    def failing(rt, meta, cache, logits_out=None):
        if torch.cuda.is_current_stream_capturing() and not state["failed"]:
            state["failed"] += 1
            raise RuntimeError("this capture fails")
        return real(rt, meta, cache, logits_out=logits_out)
    engine.model.forward = failing
    p = 10
    got = engine.step([StepEntry(slot, [tokens[p]], [0])]).cpu()               # eager
    want = plain_engine.step([StepEntry(slot0, [tokens[p]], [0])]).cpu()
    assert torch.equal(got, want)
    p += 1
    with pytest.raises(RuntimeError, match="capture fails"):                    # the capture
        engine.step([StepEntry(slot, [tokens[p]], [0])])
    assert engine.cache.length(slot) == p and engine.graphs_captured == 0
    engine.cache.check()
    for p in range(11, 40):              # eager again, then captured, then replays
        got = engine.step([StepEntry(slot, [tokens[p]], [0])]).cpu()
        want = plain_engine.step([StepEntry(slot0, [tokens[p]], [0])]).cpu()
        assert torch.equal(got, want), p
    assert state["failed"] == 1 and engine.graphs_captured == 1


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_graph_replays_equal_eager_steps(dtype, model_root):
    """Decoding through captured graphs gives, replay after replay, what eager steps give; eager
    work of other sequences (prompts, frees, a batch of another size) runs between the replays."""
    folder = make_folder(model_root, "B", dtype)
    vocab = 384
    seqs = [random_tokens(vocab, 150, 90 + i) for i in range(3)]
    other = random_tokens(vocab, 40, 99)
    outs = {}
    for graphs in (False, True):
        engine = hb.Engine.from_folder(folder, dtype=dtype, max_tokens=64 * 16, use_graphs=graphs)
        assert engine.use_graphs == graphs
        slots = [engine.alloc_slot() for _ in seqs]
        engine.step([StepEntry(s, t[:20], []) for s, t in zip(slots, seqs)])
        got = []
        for p in range(20, 150):
            if p % 37 == 0:                       # eager work in between, with a synchronisation
                extra = engine.alloc_slot()
                engine.step([StepEntry(extra, other, [39])]).cpu()
                engine.step([StepEntry(extra, [5], [0])]).cpu()
                engine.free_slot(extra)
            got.append(engine.step([StepEntry(s, [t[p]], [0]) for s, t in zip(slots, seqs)]).cpu().numpy())
        outs[graphs] = np.stack(got)
        if graphs:
            assert engine.graphs_captured > 0 and len(engine._graphs) > 0
        engine.cache.check()
    assert np.array_equal(outs[True], outs[False])
    ref = plain_logits(folder, seqs[1])
    for i, p in enumerate(range(20, 150)):
        assert close(outs[True][i][1], ref[p], dtype, "B")[0], p


@pytest.mark.parametrize("name,batch", [("D", 1), ("D", 5), ("B", 16), ("B", 17), ("D", 20)])
def test_norms_handed_from_product_to_product(name, batch, model_root, monkeypatch):
    """With at most 16 rows in bfloat16 the product that adds to the residual stream prepares the norm
    that follows and the next product finishes it: between a step's first norm and its last no
    norm kernel runs. With 17 to 64 rows a product whose K is long enough to be cut into slices norms
    the rows in the kernel that adds the slices up (model D's output projection: K = 512), and
    every other norm has its kernel again (all of model B's). Both ways give the plain
    implementation's logits, and nearly each other's (they differ in the order in which a row's
    squares are added up)."""
    from herbert_rs_amd.kernels import ops
    from herbert_rs_amd.parts.norm import RMSNorm
    folder = make_folder(model_root, name, "bfloat16")
    raw = CONFIGS[name][0]
    layers = raw["num_hidden_layers"]
    seqs = [random_tokens(raw["vocab_size"], 9 + i % 5, 300 + i) for i in range(batch)]
    calls = []
    real = ops.rmsnorm
    monkeypatch.setattr(ops, "rmsnorm", lambda *a, **k: (calls.append(1), real(*a, **k))[1])
    got = {}
    for hands_on in (True, False):
        monkeypatch.setattr(RMSNorm, "hands_on", hands_on)
        engine = hb.Engine.from_folder(folder, dtype="bfloat16", max_tokens=64 * batch, use_graphs=False)
        slots = [engine.alloc_slot() for _ in seqs]
        engine.step([StepEntry(s, t[:-1], []) for s, t in zip(slots, seqs)])
        del calls[:]
        got[hands_on] = engine.step([StepEntry(s, [t[-1]], [0]) for s, t in zip(slots, seqs)]).cpu().numpy()
        if hands_on and batch <= 16:
            assert len(calls) == 2, len(calls)              # the first layer's input norm and the final norm
        elif hands_on and name == "D":
            assert len(calls) == layers + 1, len(calls)     # no norm kernel after the output projections
        elif batch > 16:
            assert len(calls) == 2 * layers + 1, len(calls)
        else:
            assert layers + 1 <= len(calls) <= 2 * layers + 1, len(calls)
    for i, t in enumerate(seqs):
        ref = plain_logits(folder, t)[-1]
        for hands_on in (True, False):
            ok, err = close(got[hands_on][i], ref, "bfloat16", name)
            assert ok, (i, hands_on, err)
    if batch <= 16 or name == "D":
        assert float(np.abs(got[True] - got[False]).max()) <= 2 ** -7 * float(np.abs(got[False]).max())


def test_graphs_survive_larger_batches_that_outgrow_the_scratch_buffers(model_root):
    """A graph captured for two sequences keeps writing to the scratch buffers of its time. A later
    batch of nine needs larger ones: the old ones must stay allocated. Here other tensors are
    allocated and filled in between, which would land in freed memory and be overwritten by the
    graph of two when it is replayed afterwards; and that graph must still give what eager steps give."""
    folder = make_folder(model_root, "D", "bfloat16")
    vocab = CONFIGS["D"][0]["vocab_size"]
    seqs = [random_tokens(vocab, 40, 700 + i) for i in range(9)]
    outs = {}
    for graphs in (False, True):
        engine = hb.Engine.from_folder(folder, dtype="bfloat16", max_tokens=64 * 12, use_graphs=graphs)
        two = [engine.alloc_slot() for _ in range(2)]
        engine.step([StepEntry(s, seqs[i][:2], []) for i, s in enumerate(two)])          # prompts smaller than the batches
        got = [engine.step([StepEntry(s, [seqs[i][p]], [0]) for i, s in enumerate(two)]).cpu().numpy()
               for p in range(2, 8)]                                                      # captured on the second step
        more = [engine.alloc_slot() for _ in range(7)]
        engine.step([StepEntry(s, seqs[2 + i][:2], []) for i, s in enumerate(more)])
        for p in range(2, 6):
            engine.step([StepEntry(s, [seqs[2 + i][p]], [0]) for i, s in enumerate(more)] +
                        [StepEntry(s, [seqs[i][6 + p]], [0]) for i, s in enumerate(two)])   # nine rows: larger buffers
        # tensors of many small sizes: whatever was freed when the buffers grew is handed out again here
        junk = [torch.full((128 << (i % 10),), float("nan"), device="cuda") for i in range(3000)]
        torch.cuda.synchronize()
        for s in more:
            engine.free_slot(s)
        got += [engine.step([StepEntry(s, [seqs[i][p]], [0]) for i, s in enumerate(two)]).cpu().numpy()
                for p in range(12, 24)]                                                   # the graph of two again
        torch.cuda.synchronize()
        assert all(bool(torch.isnan(t).all()) for t in junk), "a replayed graph wrote into memory that was freed"
        del junk
        outs[graphs] = np.stack(got)
        if graphs:
            assert engine.graphs_captured > 0 and len(engine._graphs) > 0
        engine.cache.check()
    assert np.isfinite(outs[True]).all()
    assert np.array_equal(outs[True], outs[False])
