"""Contexts of 9,000 to 17,000 tokens against the plain implementation, through bin/trace_run.

The reference runs contexts out to 16,000 tokens (docs/benchmarks/qwen3-0.6b-results.md:41-49) and
feeds long prompts in chunks that must give what the whole prompt gives
(crates/backends/backend_common/src/generic_model.rs:445-522). Above 4,096 tokens the engine's
decode steps change the width of their context buckets (512 tokens at 6,000, 1,024 at 9,000, 2,048
at 17,000), the decode attention cuts a context into more than 32 ranges, a prompt's chunks attend over a long cache, and a batch with one long sequence
beside short ones deals the attention's grid out by a list: every one of these is crossed here, in
bfloat16 and in float32, with a model of heads of 128 and one of heads of 64.

Random weights would hide a lost page among hundreds (softmax over 17,000 keys of alike scores is
nearly their mean): the per-head norm weights of queries and keys are scaled so that scores have a
standard deviation near 3 and a handful of keys, anywhere in the context, hold most of a query's
weight. A page, a range or a chunk that went missing would then move logits by far more than the
bounds allow.
"""
import os

import numpy as np
import pytest
import torch
from safetensors.torch import load_file, save_file

from . import replay_util as ru
from .bounds import close
from .plain_cache import forget, plain_rows
from .tiny import make_folder_from, random_tokens

pytestmark = pytest.mark.gpu

# One layer each: the context's length matters to the attention and to the cache alone. Eight kv heads
# of 128: a chunk of 8,192 tokens then has enough tiles for the long-prompt attention kernel, one of
# 2,048 keeps the kernel of 32-token tiles; heads of 128 take the q/k/v product that writes the cache
# itself and the decode kernel that norms, rotates and writes. Four kv heads of 64 with two query heads
# each: the long-prompt kernel only in the step that brings a batch's four prompts at once.
LONG_128 = dict(
    architectures=["Qwen3ForCausalLM"], model_type="qwen3",
    num_hidden_layers=1, hidden_size=256, num_attention_heads=8, num_key_value_heads=8, head_dim=128,
    intermediate_size=384, vocab_size=512, rope_theta=1000000.0, rms_norm_eps=1e-6,
    tie_word_embeddings=True, max_position_embeddings=20480, eos_token_id=511)
LONG_64 = dict(
    architectures=["Qwen3ForCausalLM"], model_type="qwen3",
    num_hidden_layers=1, hidden_size=192, num_attention_heads=8, num_key_value_heads=4, head_dim=64,
    intermediate_size=256, vocab_size=320, rope_theta=500000.0, rms_norm_eps=1e-5,
    tie_word_embeddings=False, max_position_embeddings=20480, eos_token_id=3)
MODELS = {"long128": (LONG_128, 31), "long64": (LONG_64, 32)}
SCORE_SCALE = 3.0 ** 0.5        # on each of q_norm and k_norm: scores of a standard deviation near 3
DECODE_STEPS = 20


def peaked_folder(root, tag):
    """The random model `tag` (bfloat16 storage, read by both modes) with its per-head norm weights
    scaled up, written once."""
    raw, seed = MODELS[tag]
    folder = make_folder_from(root, tag, raw, seed=seed, dtype="bfloat16", std=0.05, norm_std=0.1)
    marker = os.path.join(folder, "peaked")
    if not os.path.exists(marker):
        path = os.path.join(folder, "model.safetensors")
        tensors = load_file(path)
        for name in tensors:
            if name.endswith("q_norm.weight") or name.endswith("k_norm.weight"):
                tensors[name] = (tensors[name].float() * SCORE_SCALE).to(tensors[name].dtype)
        save_file(tensors, path)
        open(marker, "w").close()
    return folder


def requests(vocab, tag):
    """id -> (tokens, prompt length, chunk of the prompt or None for "in the batch's one step")."""
    reqs = {"p9": (random_tokens(vocab, 9000 + DECODE_STEPS, 700), 9000, 2048)}
    if tag == "long128":
        reqs["p17"] = (random_tokens(vocab, 17000 + DECODE_STEPS, 701), 17000, 8192)
    else:
        reqs["p6"] = (random_tokens(vocab, 6000 + DECODE_STEPS, 702), 6000, 2048)
    # a batch of four that start together: one long, three short
    for i, n in enumerate([9300, 300, 1500, 70]):
        reqs[f"u{i}"] = (random_tokens(vocab, n + DECODE_STEPS - 3 * i, 710 + i), n, None)
    return reqs


def prompt_places(n, chunk):
    """Places of a prompt whose logits are compared: the ends of pages and chunks, the first and last."""
    places = {0, 1, 63, 64, n // 2, n - 2, n - 1}
    if chunk:
        for c in range(chunk, n, chunk):
            places.update({c - 1, c, c + 1})
    return sorted(p for p in places if 0 <= p < n)


def long_trace(reqs):
    steps = []

    def add(entries, end=()):
        steps.append({"step": len(steps), "entries": entries, "end": list(end)})

    def decode(ids):
        at = {rid: reqs[rid][1] for rid in ids}
        live = list(ids)
        while live:
            entries, end = [], []
            for rid in list(live):
                toks = reqs[rid][0]
                entries.append({"id": rid, "tokens": [toks[at[rid]]], "want": [0]})
                at[rid] += 1
                if at[rid] == len(toks):
                    end.append(rid)
                    live.remove(rid)
            add(entries, end)

    for rid in [r for r in ("p17", "p9", "p6") if r in reqs]:
        toks, n, chunk = reqs[rid]
        places = prompt_places(n, chunk)
        for a in range(0, n, chunk):
            b = min(n, a + chunk)
            add([{"id": rid, "tokens": toks[a:b], "want": [p - a for p in places if a <= p < b]}])
        decode([rid])
    batch = [r for r in reqs if r.startswith("u")]
    add([{"id": rid, "tokens": reqs[rid][0][:reqs[rid][1]], "want": prompt_places(reqs[rid][1], None)}
         for rid in batch])
    decode(batch)
    return steps


@pytest.mark.parametrize("dtype", ["bfloat16", "float32"])
@pytest.mark.parametrize("tag", ["long128", "long64"])
def test_long_contexts_in_chunks_then_decoded(tag, dtype, model_root, tmp_path):
    folder = peaked_folder(model_root, tag)
    vocab = MODELS[tag][0]["vocab_size"]
    reqs = requests(vocab, tag)
    steps = long_trace(reqs)
    out = ru.run_trace(folder, dtype, steps, str(tmp_path / "out"), ru.needed_tokens(steps), vocab, timeout=600)
    got = ru.collect(steps, out)
    wanted = {}
    for (rid, pos) in got:
        wanted.setdefault(rid, []).append(pos)
    assert set(wanted) == set(reqs)
    for rid, places in wanted.items():
        toks, n, chunk = reqs[rid]
        assert sum(p >= n for p in places) == len(toks) - n
        ref = plain_rows(folder, toks, places)
        for pos in places:
            kind = "prompt" if pos < n else "decode"
            how = "batch of unequal" if chunk is None else f"chunks of {chunk}"
            ok, err = close(got[(rid, pos)], ref[pos], dtype, "long", f"{tag} {how} {kind}")
            assert ok, f"{tag} {dtype}: request {rid} position {pos} ({how}, {kind}): error {err}"
    if dtype == "float32":
        forget(folder)


def test_the_scaled_norms_make_far_keys_count():
    """What the scaling is for, on the plain formulas alone: with scores of a standard deviation near
    3, the loss of one page of 64 keys out of 9,000 moves an output (values of unit variance) by 0.02
    or more for a sixth of the pages, and by most of a value for the worst; with plain random scores
    no page moves it by 0.02, which bfloat16 rounding would cover."""
    g = torch.Generator().manual_seed(5)
    T, hd = 9000, 128
    q = torch.randn(hd, generator=g)
    k = torch.randn(T, hd, generator=g)
    v = torch.randn(T, hd, generator=g)
    moved = {}
    for scale in (1.0, 3.0):
        s = (k @ q) * scale / hd ** 0.5
        whole = torch.softmax(s, 0) @ v
        moves = []
        for page in range(T // 64):
            keep = torch.ones(T, dtype=torch.bool)
            keep[page * 64:(page + 1) * 64] = False
            moves.append(float((torch.softmax(s[keep], 0) @ v[keep] - whole).abs().max()))
        moved[scale] = np.array(moves)
    assert moved[1.0].max() < 0.02
    assert moved[3.0].max() > 0.5 and (moved[3.0] > 0.02).sum() >= len(moved[3.0]) // 7
