"""Configurations and schedules drawn at random (fixed seeds): every size and option that
config.json gives varies at once (head sizes in steps of 16 up to 128, one to eight kv heads with
one to eight query heads each, widths and vocabularies that are no power of two, one to three
layers, windows on some layers, partial rotation, linear and yarn scaling, tied and separate
heads), and so do the requests: up to seven sequences of unequal lengths whose prompts come whole or
in pieces, then their next tokens one by one, the shorter ones ending earlier. Every position's
logits are compared with the plain implementation in float32 and in bfloat16. Six larger draws
(heads of 64 and 128, widths to 1,024, up to twelve sequences, prompts to 1,500 tokens) follow."""
import random

import numpy as np
import pytest
import torch

import herbert_rs_amd as hb
from herbert_rs_amd.engine import StepEntry

from .bounds import close
from .plain import model as plain
from .tiny import make_folder_from

pytestmark = pytest.mark.gpu


def random_config(rng):
    hd = rng.choice([16, 32, 48, 64, 80, 96, 112, 128, 128, 64])
    nkv = rng.choice([1, 1, 2, 2, 3, 4, 8])
    group = rng.choice([1, 1, 2, 3, 4, 4, 5, 8])
    hidden = rng.choice([32, 40, 64, 72, 96, 100, 128, 136, 160, 192, 256, 264, 320])
    inter = rng.choice([16, 48, 56, 64, 100, 128, 176, 224, 256, 330, 400])
    vocab = rng.choice([37, 64, 100, 255, 256, 384, 500, 777, 1024, 2000])
    layers = rng.choice([1, 2, 2, 3])
    raw = dict(architectures=["Qwen3ForCausalLM"], model_type="qwen3", num_hidden_layers=layers, hidden_size=hidden,
               num_attention_heads=nkv * group, num_key_value_heads=nkv, head_dim=hd, intermediate_size=inter,
               vocab_size=vocab, rope_theta=rng.choice([1e4, 5e5, 1e6]), rms_norm_eps=rng.choice([1e-6, 1e-5, 3e-6]),
               tie_word_embeddings=rng.random() < 0.5, max_position_embeddings=1024, eos_token_id=1)
    if rng.random() < 0.3:
        raw["sliding_window"] = rng.choice([5, 33, 64, 70, 128, 200])
        raw["layer_types"] = [rng.choice(["sliding_attention", "full_attention"]) for _ in range(layers)]
    if rng.random() < 0.2:
        raw["partial_rotary_factor"] = rng.choice([0.5, 0.25])
    r = rng.random()
    if r < 0.15:
        raw["rope_scaling"] = {"rope_type": "linear", "factor": 2.0}
    elif r < 0.3:
        raw["rope_scaling"] = {"rope_type": "yarn", "factor": 4.0, "original_max_position_embeddings": 64}
    return raw


def random_requests(rng):
    n = rng.choice([1, 1, 2, 3, 4, 5, 6, 7])          # (5 and 7 run as decode steps of 6 and 8: one padding row)
    prompts = [rng.choice([1, 2, 5, 17, 63, 64, 65, 100, 129, 200, 300]) for _ in range(n)]
    more = [rng.choice([0, 1, 3, 8, 20]) for _ in range(n)]          # tokens fed one by one after the prompt
    piece = rng.choice([None, None, 16, 64, 100])                    # prompts in pieces of this many tokens
    return prompts, more, piece


def larger_config(rng):
    """Heads of 64 and of 128 (the matrix-core attention kernels), widths of 256 to 1,024, up to eight
    kv heads with up to eight query heads each, vocabularies to 16,401."""
    hd = rng.choice([64, 128, 128])
    nkv = rng.choice([1, 2, 4, 8])
    group = rng.choice([1, 2, 4, 5, 8])
    layers = rng.choice([1, 2])
    raw = dict(architectures=["Qwen3ForCausalLM"], model_type="qwen3", num_hidden_layers=layers,
               hidden_size=rng.choice([256, 384, 512, 520, 768, 1024]), num_attention_heads=nkv * group,
               num_key_value_heads=nkv, head_dim=hd, intermediate_size=rng.choice([256, 704, 1000, 1536, 2048]),
               vocab_size=rng.choice([1000, 2048, 5000, 16384 + 17]), rope_theta=rng.choice([1e4, 1e6]),
               rms_norm_eps=rng.choice([1e-6, 1e-5]), tie_word_embeddings=rng.random() < 0.5,
               max_position_embeddings=2048, eos_token_id=1)
    if rng.random() < 0.25:
        raw["sliding_window"] = rng.choice([33, 128, 500])
        raw["layer_types"] = [rng.choice(["sliding_attention", "full_attention"]) for _ in range(layers)]
    if rng.random() < 0.15:
        raw["partial_rotary_factor"] = 0.5
    return raw


def larger_requests(rng):
    n = rng.choice([1, 2, 3, 5, 7, 9, 12])
    prompts = [rng.choice([1, 5, 63, 64, 65, 200, 256, 257, 511, 700, 1024, 1500]) for _ in range(n)]
    more = [rng.choice([0, 1, 3, 8, 20, 40]) for _ in range(n)]
    piece = rng.choice([None, None, 64, 256, 300])
    return prompts, more, piece


@pytest.mark.parametrize("seed", range(24))
def test_random_configuration_and_schedule(seed, tmp_path):
    rng = random.Random(seed)
    drawn(seed, tmp_path, random_config(rng), *random_requests(rng), bounds="random")


@pytest.mark.parametrize("seed", range(1000, 1006))
def test_larger_random_configuration_and_schedule(seed, tmp_path):
    """The same with larger draws. A draw compares thousands of rows of up to 16,401 logits, and the
    largest of so many rounding errors is further out: the bounds are those of the widest vocabulary
    (a one-off sweep of 195 such draws: 3.2e-5 at worst in float32, 0.0184 and 0.072 in bfloat16)."""
    rng = random.Random(seed)
    drawn(seed, tmp_path, larger_config(rng), *larger_requests(rng), bounds="wide")


def drawn(seed, tmp_path, raw, prompts, more, piece, bounds):
    print(f"seed {seed}: {raw} prompts {prompts} then {more} one by one, pieces of {piece}", flush=True)
    for dtype in ("float32", "bfloat16"):
        folder = make_folder_from(tmp_path, "m", raw, seed, dtype=dtype, std=0.05, norm_std=0.1)
        cfg, w = plain.read_folder(folder)
        g = torch.Generator().manual_seed(seed)
        seqs = [torch.randint(0, raw["vocab_size"], (p + m,), generator=g).tolist() for p, m in zip(prompts, more)]
        refs = [plain.forward(cfg, w, s).numpy() for s in seqs]
        engine = hb.load(folder, dtype=dtype, cache_tokens=sum(-(-len(s) // 64) * 64 for s in seqs))
        slots = [engine.alloc_slot() for _ in seqs]
        got = [np.full_like(r, np.nan) for r in refs]
        fed = [0] * len(seqs)
        while any(fed[i] < prompts[i] for i in range(len(seqs))):
            entries, places = [], []
            for i, s in enumerate(seqs):
                left = prompts[i] - fed[i]
                if left <= 0:
                    continue
                n = left if piece is None else min(piece, left)
                entries.append(StepEntry(slots[i], s[fed[i]:fed[i] + n], list(range(n))))
                places.append((i, fed[i], n))
            out = engine.step(entries).cpu().numpy()
            at = 0
            for i, p, n in places:
                got[i][p:p + n] = out[at:at + n]
                at += n
                fed[i] = p + n
        step = 0
        while True:
            live = [i for i in range(len(seqs)) if prompts[i] + step < len(seqs[i])]
            if not live:
                break
            out = engine.step([StepEntry(slots[i], [seqs[i][prompts[i] + step]], [0]) for i in live]).cpu().numpy()
            for j, i in enumerate(live):
                got[i][prompts[i] + step] = out[j]
            step += 1
        for s in slots:
            engine.free_slot(s)
        engine.cache.check()
        for i, s in enumerate(seqs):
            for t in range(len(s)):
                ok, err = close(got[i][t], refs[i][t], dtype, bounds, "drawn")
                assert ok, f"{dtype}: sequence {i}, position {t}: off by {err}"
