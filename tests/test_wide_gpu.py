"""The whole model at the layer widths that the benchmark times, against the plain implementation.

Two layers of the Qwen3-8B shape (hidden 4096, 32 query heads on 8 kv heads of 128,
intermediate 12288, vocabulary 151936, separate head), random bfloat16 weights, through
bin/trace_run in bfloat16 and in float32: prompts of 2,048, 1,024 and 512 tokens (the q/k/v product
that norms, rotates and writes the cache itself, on each of its three tile shapes; gate/up on tiles
of 256 and of 192 columns), decoding at batch 1, 8 and 64 with the kernels the
host picks for these widths by itself, and batches of unequal lengths that follow one another
in slots that were used before. Nothing is patched: what runs here is what bench.py times.
"""
import numpy as np
import pytest
import torch

import herbert_rs_amd as hb
from herbert_rs_amd.engine import StepEntry

from . import replay_util as ru
from .bounds import close
from .plain_cache import forget, plain_rows
from .tiny import make_folder_from, random_tokens

pytestmark = pytest.mark.gpu

WIDE = dict(
    architectures=["Qwen3ForCausalLM"], model_type="qwen3",
    num_hidden_layers=2, hidden_size=4096, num_attention_heads=32, num_key_value_heads=8, head_dim=128,
    intermediate_size=12288, vocab_size=151936, rope_theta=1000000.0, rms_norm_eps=1e-6,
    tie_word_embeddings=False, max_position_embeddings=4096, eos_token_id=151645)
VOCAB = WIDE["vocab_size"]


def wide_requests():
    """id -> (tokens, length of the prompt part, places of the prompt whose logits are wanted)."""
    reqs = {"long": (random_tokens(VOCAB, 2048 + 6, 900), 2048, [0, 1, 63, 64, 1023, 2047]),
            # prompts for which the host picks the tiles of 192 columns and the q/k/v tiles a head wide
            "m512": (random_tokens(VOCAB, 512 + 2, 901), 512, [0, 127, 128, 511]),
            "n1024": (random_tokens(VOCAB, 1024 + 2, 902), 1024, [0, 255, 256, 1023])}
    for i, n in enumerate([300, 64, 129, 17, 200, 77, 256, 1]):                 # a batch of 8
        extra = [4, 4, 4, 2, 4, 1, 4, 4][i]
        reqs[f"e{i}"] = (random_tokens(VOCAB, n + extra, 910 + i), n, sorted({0, n - 1}))
    for i in range(64):                                                        # a batch of 64
        n = 1 + (37 * i + 11) % 90
        extra = 3 if i % 2 else 2
        reqs[f"s{i}"] = (random_tokens(VOCAB, n + extra, 1000 + i), n, [n - 1])
    for i, n in enumerate([90, 5, 130, 64, 33, 70, 2, 191]):                    # again 8, in used slots
        reqs[f"f{i}"] = (random_tokens(VOCAB, n + 3, 1100 + i), n, [n - 1])
    return reqs


def wide_trace(reqs):
    """The long prompt alone and decoded on at batch 1; then the batches of 8, of 64 and of 8,
    each: all prompts in one step, then one token each, shorter requests ending earlier."""
    steps = []

    def run_batch(ids):
        first = {"step": len(steps), "entries": [], "end": []}
        for rid in ids:
            toks, n, want = reqs[rid]
            first["entries"].append({"id": rid, "tokens": toks[:n], "want": want})
        steps.append(first)
        at = {rid: reqs[rid][1] for rid in ids}
        live = list(ids)
        while live:
            rec = {"step": len(steps), "entries": [], "end": []}
            for rid in list(live):
                toks = reqs[rid][0]
                rec["entries"].append({"id": rid, "tokens": [toks[at[rid]]], "want": [0]})
                at[rid] += 1
                if at[rid] == len(toks):
                    rec["end"].append(rid)
                    live.remove(rid)
            steps.append(rec)

    run_batch(["long"])
    run_batch(["m512"])
    run_batch(["n1024"])
    run_batch([f"e{i}" for i in range(8)])
    run_batch([f"s{i}" for i in range(64)])
    run_batch([f"f{i}" for i in range(8)])
    return steps


@pytest.fixture(scope="module")
def wide_folder(tmp_path_factory):
    root = tmp_path_factory.mktemp("wide")
    return make_folder_from(root, "wide", WIDE, seed=8, dtype="bfloat16", std=0.02, norm_std=0.1)


def test_the_host_picks_the_profiled_kernels_for_these_widths():
    """The plans of the decode steps at batch 1, 8 and 64 for the 8B widths, by the planner's
    own codes (0 = the few-row kernel; else tile + 1000 x K slices; tiles 112 = 128 x 32,
    124 = 128 x 64, 164 = 96 x 64, 184 = 256 x 64): the kernels whose profiles lie under profiles/."""
    from herbert_rs_amd.kernels import mfma
    STORE, ADD, SWIGLU = mfma.EPI_STORE, mfma.EPI_ADD, mfma.EPI_SWIGLU
    H, Q, I, V = 4096, 6144, 12288, VOCAB
    plan = mfma.gemm_plan
    for M in (1, 8):
        assert plan(M, H, H, ADD, leaves_norm=True) == 0                       # o: few rows
        assert plan(M, H, I, ADD, leaves_norm=True) == 0                       # down
        assert plan(M, 2 * I, H, SWIGLU, finishes_norm=True) == 112            # gate/up: 128 x 32 tiles
        assert plan(M, V, H, STORE) == 0                                       # head
    assert plan(1, Q, H, STORE, finishes_norm=True, defer_slices=True) == 0    # q/k/v at batch 1
    assert plan(8, Q, H, STORE, finishes_norm=True, defer_slices=True) == 4112  # 4 K slices, added up by the attention
    assert plan(64, Q, H, STORE, defer_slices=True) == 4124
    assert plan(64, H, H, ADD, leaves_norm=True) == 8124 and plan(64, H, I, ADD, leaves_norm=True) == 8124
    assert plan(64, 2 * I, H, SWIGLU) == 164 and plan(64, V, H, STORE) == 184
    assert mfma.norm_handoff(8, H, H) == "half" and mfma.norm_handoff(64, H, I) == "whole"
    # the prompt of 2,048 tokens: the fused q/k/v product is taken from 136 tiles of 256 x 256 on
    assert -(-2048 // 256) * -(-Q // 256) >= mfma.QKV_FUSE_MIN_TILES
    assert plan(2048, 2 * I, H, SWIGLU) == 188 and plan(2048, H, I, ADD) == 142
    # prompts of 512 and 1,024 tokens: gate/up on tiles of 192 columns, q/k/v fused on tiles a head
    # wide and 128 or 256 rows high; 256 tokens are too few for a fused q/k/v product
    assert plan(512, 2 * I, H, SWIGLU) == 168 and plan(1024, 2 * I, H, SWIGLU) == 168
    assert [mfma.qkv_tile_shape(m, Q) for m in (256, 512, 1024, 2048)] == [None, 2, 1, 0]
    # rows that end just past whole tiles are cut off as a product of their own; 2,048 rows are never cut
    assert mfma.gemm_split(2048, H, I, ADD) == 0 and mfma.gemm_split(2048, 2 * I, H, SWIGLU) == 0
    assert mfma.gemm_split(2049, 2 * I, H, SWIGLU) == 2048 and mfma.gemm_split(2049, H, H, ADD) == 2048


@pytest.mark.parametrize("dtype", ["bfloat16", "float32"])
def test_prompt_of_2048_and_decoding_at_batch_1_8_64(dtype, wide_folder, tmp_path):
    reqs = wide_requests()
    steps = wide_trace(reqs)
    assert max(len(s["entries"]) for s in steps) == 64
    out = ru.run_trace(wide_folder, dtype, steps, str(tmp_path / "out"), ru.needed_tokens(steps), VOCAB,
                       timeout=600)
    got = ru.collect(steps, out)
    wanted = {}
    for (rid, pos) in got:
        wanted.setdefault(rid, []).append(pos)
    assert len(got) == sum(len(w) + len(t) - n for t, n, w in reqs.values())
    for rid, places in wanted.items():
        ref = plain_rows(wide_folder, reqs[rid][0], places)
        for pos in places:
            kind = "prompt" if pos < reqs[rid][1] else "decode"
            group = {"l": "b1", "m": "b1", "n": "b1", "e": "b8", "s": "b64", "f": "b8 again"}[rid[0]]
            ok, err = close(got[(rid, pos)], ref[pos], dtype, "wide", f"{group} {kind}")
            assert ok, f"request {rid} position {pos} ({group} {kind}): error {err}"
    if dtype == "float32":
        forget(wide_folder)


def test_decoding_at_every_batch_size_of_the_ladder_at_these_widths(wide_folder):
    """Decode steps run at a ladder of batch sizes, and the host picks other kernels along it (the
    few-row kernel up to 16 rows, tiles of 32 and of 64 rows with K slices and a second kernel that
    norms, larger tiles beyond; an RMSNorm handed on half done or whole). Every size up to 80 and three up to 256, with
    one sequence fewer than the size where that leaves a padding row, at the 8B widths: the bfloat16
    engine's logits against those of the float32 engine (which the other tests hold against the
    plain implementation), within the bounds of these widths, for the prompts' last tokens and three
    decode steps."""
    from herbert_rs_amd.engine.batch import decode_batch_bucket
    sizes = sorted({decode_batch_bucket(n) for n in range(1, 81)})
    assert sizes[:10] == [1, 2, 3, 4, 6, 8, 10, 12, 14, 16] and sizes[-1] == 80
    few_of = {144: 136, 208: 200}           # beyond 64 the ladder's steps are wider: eight rows of padding
    sizes += [144, 208, 256]
    most = max(sizes)
    engines = {d: hb.load(wide_folder, dtype=d, cache_tokens=64 * 4 * most) for d in ("bfloat16", "float32")}
    worst = 0.0
    for size in sizes:
        n = few_of.get(size, size - 1 if size in (6, 10, 14, 20, 28, 40, 56, 72) else size)      # every other size with a padding row
        assert decode_batch_bucket(n) == size
        lengths = [1 + (41 * i + 7 * size) % 150 for i in range(n)]
        seqs = [random_tokens(VOCAB, m + 3, 2000 + 97 * size + i) for i, m in enumerate(lengths)]
        outs = {}
        for d, engine in engines.items():
            slots = [engine.alloc_slot() for _ in range(n)]
            rows = [engine.step([StepEntry(s, t[:m], [m - 1]) for s, t, m in zip(slots, seqs, lengths)])]
            for j in range(3):
                rows.append(engine.step([StepEntry(s, [t[m + j]], [0]) for s, t, m in zip(slots, seqs, lengths)]))
            outs[d] = torch.stack(rows).double()                 # [4, n, vocab]
            for s in slots:
                engine.free_slot(s)
            engine.cache.check()
        ref, got = outs["float32"], outs["bfloat16"]
        rms = ref.pow(2).mean(-1).sqrt().clamp_min(1e-30)
        rel_max = ((got - ref).abs().amax(-1) / rms)
        rel_l2 = ((got - ref).pow(2).mean(-1).sqrt() / rms)
        from .bounds import BF16_REL_L2, BF16_REL_RMS
        from .conftest import observe
        observe("bfloat16 wide every size, against float32: max / rms", float(rel_max.max()))
        observe("bfloat16 wide every size, against float32: rms / rms", float(rel_l2.max()))
        assert float(rel_max.max()) <= BF16_REL_RMS["wide"] and float(rel_l2.max()) <= BF16_REL_L2["wide"], \
            (size, n, float(rel_max.max()), float(rel_l2.max()))
        worst = max(worst, float(rel_l2.max()))
    assert worst > 0.0


def test_the_whole_8b_shape_in_bfloat16_against_float32():
    """All 36 layers at the full widths, weights drawn on the GPU from a seed (as the benchmark draws
    them): the bfloat16 engine against the float32 engine on the same bfloat16-valued weights, for
    a step of eight unequal prompts and four decode steps. The rounding of thirty-six layers adds up
    (observed: 0.037 of a row's rms in the rms of the error, 0.17 in its largest entry, where two
    layers give 0.011 and 0.055); a fault in a kernel that only deep or wide models reach would
    show as an error near 1. The float32 engine itself is held against the plain implementation at
    these widths (two layers) and at this depth (a quarter of the width) by the other tests."""
    cfg = hb.Qwen3Config.from_dict(dict(WIDE, num_hidden_layers=36))
    lengths = [700, 33, 129, 5, 64, 300, 1, 250]
    seqs = [random_tokens(VOCAB, n + 4, 2500 + i) for i, n in enumerate(lengths)]
    outs = {}
    for dtype in ("bfloat16", "float32"):
        engine = hb.Engine.from_config(cfg, seed=2, dtype=dtype, weight_dtype="bfloat16", std=0.02, norm_std=0.1,
                                       max_tokens=64 * 40, max_slots=8)
        slots = [engine.alloc_slot() for _ in seqs]
        rows = [engine.step([StepEntry(s, t[:n], [n - 1]) for s, t, n in zip(slots, seqs, lengths)])]
        for j in range(4):
            rows.append(engine.step([StepEntry(s, [t[n + j]], [0]) for s, t, n in zip(slots, seqs, lengths)]))
        outs[dtype] = torch.stack(rows).double().cpu()
        engine.cache.check()
        del engine
        torch.cuda.empty_cache()
    ref, got = outs["float32"], outs["bfloat16"]
    assert bool(torch.isfinite(ref).all()) and bool(torch.isfinite(got).all())
    rms = ref.pow(2).mean(-1).sqrt()
    rel_max = float(((got - ref).abs().amax(-1) / rms).max())
    rel_l2 = float(((got - ref).pow(2).mean(-1).sqrt() / rms).max())
    from .conftest import observe
    observe("bfloat16 whole 8B shape, against float32: max / rms", rel_max)
    observe("bfloat16 whole 8B shape, against float32: rms / rms", rel_l2)
    assert rel_l2 <= 0.07 and rel_max <= 0.3, (rel_l2, rel_max)
