"""The other two shapes that the benchmark times, one layer each, and a deep model, against the
plain implementation.

One layer at the Qwen3-1.7B widths (hidden 2048, 16 query heads on 8 kv heads of 128, intermediate
6144, the 151,936-row table tied to the head) and one at the Qwen3-32B widths (hidden 5120, 64 query
heads on 8 kv heads, intermediate 25,600), through bin/trace_run in bfloat16 and float32: a prompt
of 2,048 tokens decoded on at batch 1, then a batch of the workload's size (16 and 8) with unequal
prompts. The kernels are the ones the host picks for these widths by itself; the plans are asserted
by the planner's own codes. Then 36 layers at a quarter of the 8B width: how the error grows with
depth, in float32 and in bfloat16.
"""
import json
import os

import numpy as np
import pytest

import herbert_rs_amd as hb
from herbert_rs_amd.engine import StepEntry

from . import replay_util as ru
from .bounds import close
from .conftest import observe
from .plain import model as plain
from .plain_cache import forget, plain_folder, plain_rows
from .tiny import make_folder_from, random_tokens

pytestmark = pytest.mark.gpu

VOCAB = 151936
SHAPES = {
    "1p7b": (dict(
        architectures=["Qwen3ForCausalLM"], model_type="qwen3",
        num_hidden_layers=1, hidden_size=2048, num_attention_heads=16, num_key_value_heads=8, head_dim=128,
        intermediate_size=6144, vocab_size=VOCAB, rope_theta=1000000.0, rms_norm_eps=1e-6,
        tie_word_embeddings=True, max_position_embeddings=4096, eos_token_id=151645), 16),
    # (the 32B checkpoints have a head of their own; the table doubles as head here to halve what the
    # test writes and reads: the product is the same kernel either way, and the two layers at the 8B
    # widths have the separate head)
    "32b": (dict(
        architectures=["Qwen3ForCausalLM"], model_type="qwen3",
        num_hidden_layers=1, hidden_size=5120, num_attention_heads=64, num_key_value_heads=8, head_dim=128,
        intermediate_size=25600, vocab_size=VOCAB, rope_theta=1000000.0, rms_norm_eps=1e-6,
        tie_word_embeddings=True, max_position_embeddings=4096, eos_token_id=151645), 8),
}


def shape_requests(batch):
    reqs = {"long": (random_tokens(VOCAB, 2048 + 4, 1200), 2048, [0, 1, 63, 64, 1023, 2047])}
    for i in range(batch):
        n = 1 + (53 * i + 29) % 290
        reqs[f"b{i}"] = (random_tokens(VOCAB, n + 2 + i % 3, 1210 + i), n, [n - 1])
    return reqs


def shape_trace(reqs):
    steps = []

    def run_batch(ids):
        steps.append({"step": len(steps), "end": [], "entries": [
            {"id": rid, "tokens": reqs[rid][0][:reqs[rid][1]], "want": reqs[rid][2]} for rid in ids]})
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
    run_batch([r for r in reqs if r != "long"])
    return steps


def test_the_host_picks_these_kernels_for_the_two_shapes():
    """By the planner's codes (0 = the few-row kernel; else tile + 1000 x K slices; tiles 112 = 128 x
    32, 184 = 256 x 64, 142 = 256 x 128, 168 = 192 x 256, 186 = 256 x 192, 188 = 256 x 256)."""
    from herbert_rs_amd.kernels import mfma
    STORE, ADD, SWIGLU = mfma.EPI_STORE, mfma.EPI_ADD, mfma.EPI_SWIGLU
    plan = mfma.gemm_plan
    H, Q, I = 2048, 32 * 128, 6144                       # 1.7B widths: everything of few rows is the few-row kernel
    for M in (1, 16):
        assert plan(M, Q, H, STORE, finishes_norm=True, defer_slices=True) == 0
        assert plan(M, H, H, ADD, leaves_norm=True) == 0 and plan(M, H, I, ADD, leaves_norm=True) == 0
        assert plan(M, 2 * I, H, SWIGLU, finishes_norm=True) == 0
    assert plan(1, VOCAB, H, STORE) == 0 and plan(16, VOCAB, H, STORE) == 112
    assert plan(2048, 2 * I, H, SWIGLU) == 168 and plan(2048, H, I, ADD) == 2142
    assert mfma.qkv_tile_shape(2048, Q) == 1
    H, Q, I, D = 5120, 80 * 128, 25600, 8192             # 32B widths: the tiled kernel with K slices takes over
    for M in (1, 8):
        assert plan(M, Q, H, STORE, finishes_norm=True, defer_slices=True) == 0
        assert plan(M, 2 * I, H, SWIGLU, finishes_norm=True) == 112
        assert plan(M, H, I, ADD, leaves_norm=True) == 8184
        assert plan(M, VOCAB, H, STORE) == 0
    assert plan(1, H, D, ADD, leaves_norm=True) == 0 and plan(8, H, D, ADD, leaves_norm=True) == 4112
    assert plan(2048, 2 * I, H, SWIGLU) == 188 and plan(2048, H, I, ADD) == 186
    assert mfma.qkv_tile_shape(2048, Q) == 0


@pytest.mark.parametrize("dtype", ["bfloat16", "float32"])
@pytest.mark.parametrize("shape", ["1p7b", "32b"])
def test_one_layer_at_the_widths_of_the_other_two_workloads(shape, dtype, tmp_path_factory, tmp_path):
    raw, batch = SHAPES[shape]
    root = tmp_path_factory.getbasetemp() / "shapes"
    folder = make_folder_from(root, shape, raw, seed=3 if shape == "1p7b" else 4, dtype="bfloat16", std=0.02,
                              norm_std=0.1)
    reqs = shape_requests(batch)
    steps = shape_trace(reqs)
    assert max(len(s["entries"]) for s in steps) == batch
    out = ru.run_trace(folder, dtype, steps, str(tmp_path / "out"), ru.needed_tokens(steps), VOCAB, timeout=600)
    got = ru.collect(steps, out)
    wanted = {}
    for (rid, pos) in got:
        wanted.setdefault(rid, []).append(pos)
    assert len(got) == sum(len(w) + len(t) - n for t, n, w in reqs.values())
    for rid, places in wanted.items():
        ref = plain_rows(folder, reqs[rid][0], places)
        for pos in places:
            kind = "prompt" if pos < reqs[rid][1] else "decode"
            group = "b1" if rid == "long" else f"b{batch}"
            ok, err = close(got[(rid, pos)], ref[pos], dtype, "wide", f"{shape} {group} {kind}")
            assert ok, f"{shape} {dtype}: request {rid} position {pos} ({group} {kind}): error {err}"
    if dtype == "float32":
        forget(folder)
        os.remove(os.path.join(folder, "model.safetensors"))


DEEP = dict(
    architectures=["Qwen3ForCausalLM"], model_type="qwen3",
    num_hidden_layers=36, hidden_size=1024, num_attention_heads=8, num_key_value_heads=2, head_dim=128,
    intermediate_size=3072, vocab_size=4096, rope_theta=1000000.0, rms_norm_eps=1e-6,
    tie_word_embeddings=False, max_position_embeddings=1024, eos_token_id=1)
DEPTHS = (1, 2, 4, 9, 18, 36)
_plain_by_depth = {}


def folder_of_depth(deep_folder, layers):
    """The deep model's first `layers` layers as a model folder of its own: the same tensors (stored
    tensors that a model does not ask for are passed over), another config.json."""
    folder = f"{deep_folder}_first{layers}"
    if not os.path.exists(folder):
        os.makedirs(folder)
        with open(os.path.join(folder, "config.json"), "w") as f:
            json.dump(dict(DEEP, num_hidden_layers=layers), f)
        os.symlink(os.path.join(deep_folder, "model.safetensors"), os.path.join(folder, "model.safetensors"))
    return folder


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_error_by_depth_up_to_36_layers(dtype, tmp_path_factory):
    """A prompt of 200 tokens, eight single tokens, and a batch of four unequal sequences, through
    models of 1 to 36 layers. The worst error at each depth is printed with the run's summary; the
    float32 bound and the bfloat16 bounds hold at every depth."""
    root = tmp_path_factory.getbasetemp() / "deep"
    deep = make_folder_from(root, "deep", DEEP, seed=36, dtype="bfloat16", std=0.02, norm_std=0.1)
    vocab = DEEP["vocab_size"]
    seqs = [random_tokens(vocab, n, 1300 + i) for i, n in enumerate([208, 90, 17, 150, 65])]
    cfg, w = plain_folder(deep)
    for layers in DEPTHS:
        folder = folder_of_depth(deep, layers)
        engine = hb.load(folder, dtype=dtype, cache_tokens=64 * 12)
        if layers not in _plain_by_depth:
            _plain_by_depth[layers] = [plain.forward(dict(cfg, num_hidden_layers=layers), w, t).numpy() for t in seqs]
        ref = _plain_by_depth[layers]
        got = [[] for _ in seqs]
        slot = engine.alloc_slot()
        got[0].extend(engine.step([StepEntry(slot, seqs[0][:200], list(range(200)))]).cpu().numpy())
        for p in range(200, 208):
            got[0].extend(engine.step([StepEntry(slot, [seqs[0][p]], [0])]).cpu().numpy())
        engine.free_slot(slot)
        slots = [engine.alloc_slot() for _ in seqs[1:]]
        heads = [len(t) - 6 for t in seqs[1:]]
        rows = engine.step([StepEntry(s, t[:h], list(range(h))) for s, t, h in zip(slots, seqs[1:], heads)]).cpu().numpy()
        at = 0
        for i, h in enumerate(heads):
            got[1 + i].extend(rows[at:at + h])
            at += h
        for p in range(6):
            rows = engine.step([StepEntry(s, [t[h + p]], [0]) for s, t, h in zip(slots, seqs[1:], heads)]).cpu().numpy()
            for i in range(len(slots)):
                got[1 + i].append(rows[i].copy())
        for s in slots:
            engine.free_slot(s)
        engine.cache.check()
        worst = 0.0
        for i, t in enumerate(seqs):
            assert len(got[i]) == len(t)
            for p in range(len(t)):
                ok, err = close(got[i][p], ref[i][p], dtype, "deep", f"{layers:2d} layers")
                worst = max(worst, err)
                assert ok, f"{dtype}, {layers} layers: sequence {i} position {p}: error {err}"
            observe(f"{dtype} deep {layers:2d} layers: rms of a row of plain logits",
                    float(np.sqrt((ref[i].astype(np.float64) ** 2).mean())))
        del engine
    if dtype == "bfloat16":
        forget(deep)
        _plain_by_depth.clear()
