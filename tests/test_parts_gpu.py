"""Each part alone against the plain formulas, models put together from parts in other ways
(a layer run twice, a layer that reads another's cache, no rotation), and a toy mixer with state
of its own, a toy feed-forward with routing and two toy position encodings (another rotation
table; learned rows added to the embedding, no rotation at all), a toy arrangement of a layer and a
toy norm that are registered here, outside the framework's files."""
import numpy as np
import pytest
import torch

from herbert_rs_amd.cache import Cache, KVNeed, StateNeed
from herbert_rs_amd.engine import Engine, StepEntry
from herbert_rs_amd.engine import batch as batching
from herbert_rs_amd.engine.model import SharedParts
from herbert_rs_amd.parts.attention import Attention
from herbert_rs_amd.parts import (LayerSpec, ModelSpec, Part, PartSpec, Runtime, ScheduleEntry, StepContext,
                                  build, register)
from herbert_rs_amd.weights import TensorNeed

from .plain import ops as pops

pytestmark = pytest.mark.gpu
DEV = "cuda"


def rand(*shape, seed=0, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return torch.randn(*shape, generator=g) * scale


def context(needs, lengths_new, dtype=torch.float32, max_positions=256):
    """(ctx, cache, slots) for sequences that bring lengths_new[i] tokens to fresh slots."""
    rt = Runtime(dtype, DEV)
    cache = Cache(needs, 64 * 8, max_positions, dtype, DEV)
    slots = [cache.alloc_slot() for _ in lengths_new]
    entries = [StepEntry(s, [0] * n, []) for s, n in zip(slots, lengths_new)]
    for e in entries:
        cache.reserve(e.slot, len(e.tokens))
    meta = batching.pack(entries, [0] * len(entries), torch.device(DEV))
    return StepContext(rt=rt, meta=meta, cache=cache), cache, slots


def test_norm_part():
    w = 1 + 0.1 * rand(96, seed=1)
    part = build("norm", PartSpec("rmsnorm", {"size": 96, "eps": 1e-5, "weight": "n.weight"}))
    assert part.tensor_needs() == {"n.weight": TensorNeed((96,), "scale")}
    rt = Runtime(torch.float32, DEV)
    part.load({"n.weight": w}, rt)
    x = rand(5, 96, seed=2, scale=3.0)
    ctx = StepContext(rt=rt, meta=None, cache=None)
    got = part.forward(ctx, x.to(DEV)).cpu()
    assert torch.allclose(got, pops.rms_norm(x, w, 1e-5), atol=1e-5)
    rows = torch.tensor([4, 1], dtype=torch.int32, device=DEV)
    assert torch.allclose(part.forward(ctx, x.to(DEV), rows).cpu(), pops.rms_norm(x[[4, 1]], w, 1e-5), atol=1e-5)


def test_position_part_tables():
    part = build("position", PartSpec("rope", {"theta": 1e6, "rotary_dims": 32, "max_positions": 100}))
    part.load({}, Runtime(torch.float32, DEV))
    cos, sin, rot = part.rotation()
    pc, ps = pops.rope_tables(list(range(100)), 32, 1e6)
    assert rot == 32 and torch.equal(cos.cpu(), pc) and torch.equal(sin.cpu(), ps)
    assert build("position", PartSpec("none")).rotation() is None
    for scaling, plain_scaling in ((("linear", 4.0, None, 32.0, 1.0), {"type": "linear", "factor": 4.0}),
                                   (("yarn", 8.0, 40, 16.0, 2.0), {"type": "yarn", "factor": 8.0, "beta_fast": 16.0,
                                                                   "original_max_position_embeddings": 40, "beta_slow": 2.0}),
                                   (("yarn", 2.0, None, 32.0, 1.0), {"type": "yarn", "factor": 2.0, "beta_fast": 32.0,
                                                                     "original_max_position_embeddings": 100, "beta_slow": 1.0})):
        part = build("position", PartSpec("rope", {"theta": 1e4, "rotary_dims": 32, "max_positions": 100, "scaling": scaling}))
        part.load({}, Runtime(torch.float32, DEV))
        cos, sin, _ = part.rotation()
        pc, ps = pops.rope_tables(list(range(100)), 32, 1e4, plain_scaling)
        assert torch.allclose(cos.cpu(), pc, atol=2e-6) and torch.allclose(sin.cpu(), ps, atol=2e-6), scaling


ATT = dict(hidden_size=40, num_heads=6, num_kv_heads=2, head_dim=16, eps=1e-6)
NAMES = {k: f"a.{k}" for k in ("q", "k", "v", "o", "q_norm", "k_norm")}


def attention_weights(seed=3, hidden=40, nq=6, nkv=2, hd=16):
    return {"a.q": rand(nq * hd, hidden, seed=seed, scale=0.2), "a.k": rand(nkv * hd, hidden, seed=seed + 1, scale=0.2),
            "a.v": rand(nkv * hd, hidden, seed=seed + 2, scale=0.2), "a.o": rand(hidden, nq * hd, seed=seed + 3, scale=0.2),
            "a.q_norm": 1 + 0.1 * rand(hd, seed=seed + 4), "a.k_norm": 1 + 0.1 * rand(hd, seed=seed + 5)}


def plain_attention(w, y, positions, theta, eps, nq, nkv, hd, qk_norm=True, rope=True, window=None):
    q = pops.split_heads(pops.linear(y, w["a.q"]), nq, hd)
    k = pops.split_heads(pops.linear(y, w["a.k"]), nkv, hd)
    v = pops.split_heads(pops.linear(y, w["a.v"]), nkv, hd)
    if qk_norm:
        q, k = pops.head_rms_norm(q, w["a.q_norm"], eps), pops.head_rms_norm(k, w["a.k_norm"], eps)
    if rope:
        q, k = pops.apply_rope(q, positions, theta), pops.apply_rope(k, positions, theta)
    a = pops.causal_attention(q, k, v, positions, window=window)
    return pops.linear(a.reshape(len(positions), nq * hd), w["a.o"])


@pytest.mark.parametrize("qk_norm,rope,window", [(True, True, None), (False, True, None), (True, False, None),
                                                 (True, True, 5)])
def test_attention_part(qk_norm, rope, window):
    pos_spec = PartSpec("rope", {"theta": 1e4, "rotary_dims": 16, "max_positions": 256}) if rope else PartSpec("none")
    names = NAMES if qk_norm else {k: v for k, v in NAMES.items() if "norm" not in k}
    part = build("mixer", PartSpec("attention", dict(ATT, position=pos_spec, names=names, qk_norm=qk_norm,
                                                     window=window)), shared=SharedParts())
    assert part.cache_need() == KVNeed(2, 16, window)
    w = attention_weights()
    assert set(part.tensor_needs()) == set(names.values())
    ctx, cache, slots = context({0: part.cache_need()}, [9, 4])
    part.position.load({}, ctx.rt)
    part.load(w, ctx.rt)
    y = rand(13, 40, seed=9)
    x = torch.zeros(13, 40, device=DEV)
    part.forward(ctx, y.to(DEV), x)
    for a, b in ((0, 9), (9, 13)):
        want = plain_attention(w, y[a:b], list(range(b - a)), 1e4, 1e-6, 6, 2, 16, qk_norm, rope, window)
        assert torch.allclose(x[a:b].cpu(), want, atol=2e-5), (a, b)


def test_feed_forward_part():
    part = build("feed_forward", PartSpec("swiglu", {"hidden_size": 40, "intermediate_size": 72,
                                                     "names": {"gate": "g", "up": "u", "down": "d"}}))
    w = {"g": rand(72, 40, seed=1, scale=0.3), "u": rand(72, 40, seed=2, scale=0.3), "d": rand(40, 72, seed=3, scale=0.3)}
    rt = Runtime(torch.float32, DEV)
    part.load(w, rt)
    y = rand(7, 40, seed=4)
    x0 = rand(7, 40, seed=5)
    x = x0.clone().to(DEV)
    part.forward(StepContext(rt=rt, meta=None, cache=None), y.to(DEV), x)
    assert torch.allclose(x.cpu(), x0 + pops.swiglu_mlp(y, w["g"], w["u"], w["d"]), atol=2e-5)


def test_embedding_and_head_parts():
    table = rand(50, 24, seed=1)
    emb = build("embedding", PartSpec("table", {"vocab_size": 50, "hidden_size": 24, "weight": "e"}))
    rt = Runtime(torch.float32, DEV)
    emb.load({"e": table}, rt)
    ids = torch.tensor([3, 49, 0], dtype=torch.int32, device=DEV)
    ctx = StepContext(rt=rt, meta=None, cache=None)
    x = emb.forward(ctx, ids)
    assert torch.equal(x.cpu(), table[[3, 49, 0]])
    nw = 1 + 0.1 * rand(24, seed=2)
    for tied in (True, False):
        norm = build("norm", PartSpec("rmsnorm", {"size": 24, "eps": 1e-6, "weight": "n"}))
        head = build("head", PartSpec("linear", {"vocab_size": 50, "hidden_size": 24, "weight": "h",
                                                 "tied_to_embedding": tied}), norm=norm)
        assert ("h" in head.tensor_needs()) == (not tied)
        hw = rand(50, 24, seed=3)
        head.load({"n": nw, "h": hw}, rt, embedding=emb)
        rows = torch.tensor([2, 0], dtype=torch.int32, device=DEV)
        got = head.forward(ctx, x, rows).cpu()
        want = pops.linear(pops.rms_norm(table[[0, 3]], nw, 1e-6), table if tied else hw)
        assert torch.allclose(got, want, atol=1e-5)


# ---- models put together in other ways
def small_spec(layers, schedule, hidden=40, vocab=60, rope=True, share_from=None, nq=4, nkv=2, hd=16):
    pos = PartSpec("rope", {"theta": 1e4, "rotary_dims": hd, "max_positions": 256}) if rope else PartSpec("none")
    specs = []
    for i in range(layers):
        p = f"L{i}."
        reads = share_from is not None and i in share_from
        names = {k: p + k for k in (("q", "o", "q_norm") if reads else ("q", "k", "v", "o", "q_norm", "k_norm"))}
        mixer = PartSpec("attention", dict(hidden_size=hidden, num_heads=nq, num_kv_heads=nkv, head_dim=hd, eps=1e-6,
                                           position=pos, names=names, reads_cache_only=reads))
        ffn = PartSpec("swiglu", {"hidden_size": hidden, "intermediate_size": 56,
                                  "names": {"gate": p + "g", "up": p + "u", "down": p + "d"}})
        norms = {"input": PartSpec("rmsnorm", {"size": hidden, "eps": 1e-6, "weight": p + "n1"}),
                 "post_mixer": PartSpec("rmsnorm", {"size": hidden, "eps": 1e-6, "weight": p + "n2"})}
        specs.append(LayerSpec(PartSpec("prenorm"), mixer, ffn, norms))
    return ModelSpec(hidden_size=hidden, vocab_size=vocab, max_positions=256,
                     embedding=PartSpec("table", {"vocab_size": vocab, "hidden_size": hidden, "weight": "emb"}),
                     layers=specs, schedule=schedule,
                     final_norm=PartSpec("rmsnorm", {"size": hidden, "eps": 1e-6, "weight": "fn"}),
                     head=PartSpec("linear", {"vocab_size": vocab, "hidden_size": hidden, "weight": "head",
                                              "tied_to_embedding": True}))


def weights_for(spec, seed=0):
    from herbert_rs_amd.engine.model import Model
    from herbert_rs_amd.weights import random_tensors
    return random_tensors(Model(spec).tensor_needs(), seed, "float32", std=0.15, norm_std=0.1)


def plain_layer(w, p, x, positions, k_v_from=None, rope=True, nq=4, nkv=2, hd=16):
    """One pre-norm layer of the small model by the plain formulas; returns (x, (k, v))."""
    y = pops.rms_norm(x, w[p + "n1"], 1e-6)
    q = pops.head_rms_norm(pops.split_heads(pops.linear(y, w[p + "q"]), nq, hd), w[p + "q_norm"], 1e-6)
    if rope:
        q = pops.apply_rope(q, positions, 1e4)
    if k_v_from is None:
        k = pops.head_rms_norm(pops.split_heads(pops.linear(y, w[p + "k"]), nkv, hd), w[p + "k_norm"], 1e-6)
        if rope:
            k = pops.apply_rope(k, positions, 1e4)
        v = pops.split_heads(pops.linear(y, w[p + "v"]), nkv, hd)
    else:
        k, v = k_v_from
    a = pops.causal_attention(q, k, v, positions).reshape(len(positions), nq * hd)
    x = x + pops.linear(a, w[p + "o"])
    y = pops.rms_norm(x, w[p + "n2"], 1e-6)
    return x + pops.swiglu_mlp(y, w[p + "g"], w[p + "u"], w[p + "d"]), (k, v)


def run_engine(spec, w, tokens, cut=None):
    engine = Engine(None, spec, w, dtype="float32", max_tokens=256)
    s = engine.alloc_slot()
    if cut is None:
        return engine.step([StepEntry(s, tokens, list(range(len(tokens))))]).cpu()
    a = engine.step([StepEntry(s, tokens[:cut], list(range(cut)))]).cpu()
    rest = [engine.step([StepEntry(s, [t], [0])]).cpu() for t in tokens[cut:]]
    return torch.cat([a] + rest)


def test_a_layer_named_twice_and_a_layer_that_reads_another_s_cache():
    # entry 0: layer 0; entry 1: layer 1 reading entry 0's keys and values; entry 2: layer 0 again
    spec = small_spec(2, [ScheduleEntry(0), ScheduleEntry(1, cache=0), ScheduleEntry(0)], share_from={1})
    w = weights_for(spec)
    tokens = [5, 9, 33, 2, 41, 17, 8]
    pos = list(range(len(tokens)))
    x = pops.embedding(tokens, w["emb"])
    x, kv0 = plain_layer(w, "L0.", x, pos)
    x, _ = plain_layer(w, "L1.", x, pos, k_v_from=kv0)
    x, _ = plain_layer(w, "L0.", x, pos)
    want = pops.linear(pops.rms_norm(x, w["fn"], 1e-6), w["emb"])
    assert torch.allclose(run_engine(spec, w, tokens), want, atol=1e-4)
    assert torch.allclose(run_engine(spec, w, tokens, cut=3), want, atol=1e-4)     # and from the cache
    from herbert_rs_amd.engine.model import Model
    assert sorted(Model(spec).cache_needs()) == [0, 2]                             # two caches, not three
    assert "L1.k" not in Model(spec).tensor_needs()


MIXED_LAYERS = {
    "float32": (40, [dict(nq=4, nkv=2, hd=16, rot=16, theta=1e4, inter=56), dict(nq=6, nkv=3, hd=32, rot=8, theta=1e6, inter=24)]),
    # (heads of 128 and of 64, rotated whole: the matrix-core kernels of both sizes in one model)
    "bfloat16": (128, [dict(nq=4, nkv=2, hd=128, rot=128, theta=1e4, inter=256), dict(nq=6, nkv=3, hd=64, rot=64, theta=1e6, inter=96)]),
}


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_layers_with_heads_of_different_sizes_and_numbers(dtype):
    """Layer 0 has 4 query and 2 kv heads, layer 1 has 6 and 3 of another size with another rotation
    and a feed-forward of another width: every part has its sizes as parameters, and the cache
    keeps the two layers' keys and values in two groups with page tables of their own."""
    from .bounds import close
    vocab = 60
    hidden, sizes = MIXED_LAYERS[dtype]
    layers = []
    for i, z in enumerate(sizes):
        p = f"L{i}."
        pos = PartSpec("rope", {"theta": z["theta"], "rotary_dims": z["rot"], "max_positions": 256})
        mixer = PartSpec("attention", dict(hidden_size=hidden, num_heads=z["nq"], num_kv_heads=z["nkv"], head_dim=z["hd"],
                                           eps=1e-6, position=pos,
                                           names={k: p + k for k in ("q", "k", "v", "o", "q_norm", "k_norm")}))
        ffn = PartSpec("swiglu", {"hidden_size": hidden, "intermediate_size": z["inter"],
                                  "names": {"gate": p + "g", "up": p + "u", "down": p + "d"}})
        norms = {"input": PartSpec("rmsnorm", {"size": hidden, "eps": 1e-6, "weight": p + "n1"}),
                 "post_mixer": PartSpec("rmsnorm", {"size": hidden, "eps": 1e-6, "weight": p + "n2"})}
        layers.append(LayerSpec(PartSpec("prenorm"), mixer, ffn, norms))
    base = small_spec(1, [ScheduleEntry(0)], hidden=hidden)
    spec = ModelSpec(hidden_size=hidden, vocab_size=vocab, max_positions=256, embedding=base.embedding, layers=layers,
                     schedule=[ScheduleEntry(0), ScheduleEntry(1), ScheduleEntry(0)], final_norm=base.final_norm,
                     head=base.head)
    from herbert_rs_amd.engine.model import Model
    from herbert_rs_amd.weights import random_tensors
    w = random_tensors(Model(spec).tensor_needs(), 21, "float32", std=0.15 if dtype == "float32" else 0.05, norm_std=0.1)
    w = {k: v.to(torch.bfloat16).float() if v.dim() == 2 else v for k, v in w.items()}      # both dtypes run the same model
    g = torch.Generator().manual_seed(21)
    seqs = [torch.randint(0, vocab, (n,), generator=g).tolist() for n in (70, 9, 130, 3, 64)]

    def plain(tokens):
        positions = list(range(len(tokens)))
        x = pops.embedding(tokens, w["emb"])
        for i in (0, 1, 0):
            z, p = sizes[i], f"L{i}."
            y = pops.rms_norm(x, w[p + "n1"], 1e-6)
            q = pops.head_rms_norm(pops.split_heads(pops.linear(y, w[p + "q"]), z["nq"], z["hd"]), w[p + "q_norm"], 1e-6)
            k = pops.head_rms_norm(pops.split_heads(pops.linear(y, w[p + "k"]), z["nkv"], z["hd"]), w[p + "k_norm"], 1e-6)
            q = pops.apply_rope(q, positions, z["theta"], rotary_ndims=z["rot"])
            k = pops.apply_rope(k, positions, z["theta"], rotary_ndims=z["rot"])
            v = pops.split_heads(pops.linear(y, w[p + "v"]), z["nkv"], z["hd"])
            a = pops.causal_attention(q, k, v, positions).reshape(len(tokens), z["nq"] * z["hd"])
            x = x + pops.linear(a, w[p + "o"])
            x = x + pops.swiglu_mlp(pops.rms_norm(x, w[p + "n2"], 1e-6), w[p + "g"], w[p + "u"], w[p + "d"])
        return pops.linear(pops.rms_norm(x, w["fn"], 1e-6), w["emb"])

    engine = Engine(None, spec, w, dtype=dtype, max_tokens=64 * 9)
    assert sorted((n.kv_heads, n.head_dim) for n in engine.cache.kv_groups) == sorted((z["nkv"], z["hd"]) for z in sizes)
    assert sorted(len(grp.entries) for grp in engine.cache.kv_groups.values()) == [1, 2]
    # the five together (decode steps of six rows): prompts less their last two tokens in one step, then one token each
    slots = [engine.alloc_slot() for _ in seqs]
    first = engine.step([StepEntry(s, t[:-2], list(range(len(t) - 2))) for s, t in zip(slots, seqs)]).cpu()
    rows, at = [], 0
    for t in seqs:
        rows.append([first[at:at + len(t) - 2]])
        at += len(t) - 2
    for j in range(2, 0, -1):
        out = engine.step([StepEntry(s, [t[len(t) - j]], [0]) for s, t in zip(slots, seqs)]).cpu()
        for i in range(len(seqs)):
            rows[i].append(out[i:i + 1])
    for i, t in enumerate(seqs):
        got, want = torch.cat(rows[i]).numpy(), plain(t).numpy()
        for p in range(len(t)):
            ok, err = close(got[p], want[p], dtype, "random", "mixed layers")
            assert ok, (i, p, err)
    for s in slots:
        engine.free_slot(s)
    engine.cache.check()


@pytest.mark.parametrize("hd", [128, 64])
def test_a_layer_that_reads_another_s_cache_in_bfloat16(hd):
    """The same schedule (layer 0, layer 1 on layer 0's keys and values, layer 0 again) in bfloat16
    with heads that the matrix-core kernels take: the layer without keys of its own norms and
    rotates its queries alone and attends over pages that another entry wrote, for prompts and for
    single tokens (four sequences together, and a fifth row of padding when one has ended)."""
    from .bounds import close
    from herbert_rs_amd.engine.model import Model
    from herbert_rs_amd.weights import random_tensors
    nq, nkv, hidden = 6, 2, 128
    spec = small_spec(2, [ScheduleEntry(0), ScheduleEntry(1, cache=0), ScheduleEntry(0)], hidden=hidden, share_from={1},
                      nq=nq, nkv=nkv, hd=hd)
    w = random_tensors(Model(spec).tensor_needs(), 31, "float32", std=0.05, norm_std=0.1)
    w = {k: v.to(torch.bfloat16).float() if v.dim() == 2 else v for k, v in w.items()}
    g = torch.Generator().manual_seed(31)
    lengths, more = [70, 5, 129, 33, 64, 2], [6, 6, 6, 6, 6, 3]
    seqs = [torch.randint(0, 60, (n + m,), generator=g).tolist() for n, m in zip(lengths, more)]
    engine = Engine(None, spec, w, dtype="bfloat16", max_tokens=64 * 10)
    assert sorted(engine.model.cache_needs()) == [0, 2]
    slots = [engine.alloc_slot() for _ in seqs]
    first = engine.step([StepEntry(s, t[:n], list(range(n))) for s, t, n in zip(slots, seqs, lengths)]).cpu()
    rows, at = [], 0
    for n in lengths:
        rows.append([first[at:at + n]])
        at += n
    for step in range(max(more)):
        live = [i for i in range(len(seqs)) if step < more[i]]          # six, then five: steps of six rows
        out = engine.step([StepEntry(slots[i], [seqs[i][lengths[i] + step]], [0]) for i in live]).cpu()
        for r, i in enumerate(live):
            rows[i].append(out[r:r + 1])
    assert engine.graphs_captured >= 1
    for i, t in enumerate(seqs):
        pos = list(range(len(t)))
        x = pops.embedding(t, w["emb"])
        x, kv0 = plain_layer(w, "L0.", x, pos, nq=nq, nkv=nkv, hd=hd)
        x, _ = plain_layer(w, "L1.", x, pos, k_v_from=kv0, nq=nq, nkv=nkv, hd=hd)
        x, _ = plain_layer(w, "L0.", x, pos, nq=nq, nkv=nkv, hd=hd)
        want = pops.linear(pops.rms_norm(x, w["fn"], 1e-6), w["emb"]).numpy()
        got = torch.cat(rows[i]).numpy()
        for p in pos:
            ok, err = close(got[p], want[p], "bfloat16", "random", "shared cache")
            assert ok, (i, p, err)


def test_a_model_without_rotation():
    spec = small_spec(1, [ScheduleEntry(0)], rope=False)
    w = weights_for(spec, seed=4)
    tokens = [1, 2, 3, 4, 5]
    x = pops.embedding(tokens, w["emb"])
    x, _ = plain_layer(w, "L0.", x, list(range(5)), rope=False)
    want = pops.linear(pops.rms_norm(x, w["fn"], 1e-6), w["emb"])
    assert torch.allclose(run_engine(spec, w, tokens, cut=2), want, atol=1e-4)


# ---- a toy mixer with state of its own, defined here
@register("mixer", "toy_decay")
class ToyDecayMixer(Part):
    """s_t = decay * s_{t-1} + W y_t ; the mixer's output is s_t. The state s lives in the cache's
    fixed-size area, one vector per sequence; it has no keys or values. It loops on the host,
    so it is not graph_safe (the default) and the engine runs its steps eagerly."""

    def __init__(self, hidden_size, decay, weight, shared=None):
        self.hidden_size, self.decay, self.weight_name = hidden_size, decay, weight
        self.w = None

    def tensor_needs(self):
        return {self.weight_name: TensorNeed((self.hidden_size, self.hidden_size))}

    def cache_need(self):
        return StateNeed((self.hidden_size,), torch.float32)

    def load(self, tensors, rt):
        self.w = tensors[self.weight_name].to(rt.device).float()

    def forward(self, ctx, y, x):
        state = ctx.cache.state_views(ctx.cache_entry)[0]          # [slots, hidden]
        meta = ctx.meta
        proj = y.float() @ self.w.T
        starts = meta.host_starts
        slots = meta.slots.tolist()
        for i in range(meta.num_seqs):
            s = state[slots[i]]
            for t in range(int(starts[i]), int(starts[i + 1])):
                s = self.decay * s + proj[t]
                x[t] += s
            state[slots[i]] = s


def toy_spec():
    """Three runs: the toy layer, an attention layer, the toy layer again (with a state of its own)."""
    layer = LayerSpec(PartSpec("prenorm"),
                      PartSpec("toy_decay", {"hidden_size": 40, "decay": 0.8, "weight": "T.mix"}),
                      PartSpec("swiglu", {"hidden_size": 40, "intermediate_size": 56,
                                          "names": {"gate": "T.g", "up": "T.u", "down": "T.d"}}),
                      {"input": PartSpec("rmsnorm", {"size": 40, "eps": 1e-6, "weight": "T.n1"}),
                       "post_mixer": PartSpec("rmsnorm", {"size": 40, "eps": 1e-6, "weight": "T.n2"})})
    base = small_spec(1, [ScheduleEntry(0)])
    return ModelSpec(hidden_size=40, vocab_size=60, max_positions=256, embedding=base.embedding,
                     layers=[layer, base.layers[0]],
                     schedule=[ScheduleEntry(0), ScheduleEntry(1), ScheduleEntry(0)],
                     final_norm=base.final_norm, head=base.head)


def plain_toy_layer(w, x):
    proj = pops.linear(pops.rms_norm(x, w["T.n1"], 1e-6), w["T.mix"])
    s, out = torch.zeros(40), []
    for j in range(x.shape[0]):
        s = 0.8 * s + proj[j]
        out.append(s)
    x = x + torch.stack(out)
    return x + pops.swiglu_mlp(pops.rms_norm(x, w["T.n2"], 1e-6), w["T.g"], w["T.u"], w["T.d"])


def test_toy_mixer_with_state_is_registered_built_and_stepped():
    spec = toy_spec()
    from herbert_rs_amd.engine.model import Model
    from herbert_rs_amd.weights import random_tensors
    model = Model(spec)
    needs = model.tensor_needs()
    assert "T.mix" in needs and model.cache_needs()[0] == StateNeed((40,), torch.float32)
    assert isinstance(model.cache_needs()[1], KVNeed)
    w = random_tensors(needs, 3, "float32", std=0.15, norm_std=0.1)
    engine = Engine(None, spec, w, dtype="float32", max_tokens=256)
    # the two runs of the toy layer (entries 0 and 2) have states of their own in one group
    assert len(engine.cache.state_groups) == 1
    assert next(iter(engine.cache.state_groups.values())).entries == [0, 2]

    seqs = [[5, 9, 33, 2, 41, 17, 8, 11], [7, 3, 50]]
    slots = [engine.alloc_slot() for _ in seqs]
    whole = engine.step([StepEntry(s, t, list(range(len(t)))) for s, t in zip(slots, seqs)]).cpu()
    for s in slots:
        engine.free_slot(s)
    # the same sequences again in the same slots, cut differently: the state must start at zero
    slots = [engine.alloc_slot() for _ in seqs]
    first = engine.step([StepEntry(s, t[:2], [0, 1]) for s, t in zip(slots, seqs)]).cpu()
    rows = {0: [first[0], first[1]], 1: [first[2], first[3]]}
    step = 2
    while any(step < len(t) for t in seqs):
        live = [i for i, t in enumerate(seqs) if step < len(t)]
        out = engine.step([StepEntry(slots[i], [seqs[i][step]], [0]) for i in live]).cpu()
        for r, i in enumerate(live):
            rows[i].append(out[r])
        step += 1
    again = torch.stack(rows[0] + rows[1])
    assert torch.allclose(again, whole, atol=1e-4)

    # and against the plain formulas
    at = 0
    for t in seqs:
        x = plain_toy_layer(w, pops.embedding(t, w["emb"]))
        x, _ = plain_layer(w, "L0.", x, list(range(len(t))))
        x = plain_toy_layer(w, x)
        want = pops.linear(pops.rms_norm(x, w["fn"], 1e-6), w["emb"])
        assert torch.allclose(whole[at:at + len(t)], want, atol=1e-4)
        at += len(t)


def test_a_step_that_fails_leaves_the_state_as_it_was():
    """The toy layer runs twice in the schedule. A step whose forward pass fails after the first run
    has changed its state (here: the second run's mixer raises) leaves every slot's state, length
    and pages as they were: the same step, run again, gives what it gives on a cache that never
    saw the failure."""
    from herbert_rs_amd.weights import random_tensors
    from herbert_rs_amd.engine.model import Model
    spec = toy_spec()
    w = random_tensors(Model(spec).tensor_needs(), 3, "float32", std=0.15, norm_std=0.1)
    seqs = [[5, 9, 33, 2, 41, 17, 8, 11], [7, 3, 50, 1]]

    def run(fail_once):
        engine = Engine(None, spec, w, dtype="float32", max_tokens=256)
        slots = [engine.alloc_slot() for _ in seqs]
        engine.step([StepEntry(s, t[:3], []) for s, t in zip(slots, seqs)])
        if fail_once:
            mixer = engine.model.blocks[0].mixer
            real, calls = mixer.forward, []

            def failing(ctx, y, x):
                calls.append(ctx.entry)
                if ctx.entry == 2:
                    raise RuntimeError("the second run fails")
                return real(ctx, y, x)
            mixer.forward = failing
            before = [g.data.clone() for g in engine.cache.state_groups.values()]
            with pytest.raises(RuntimeError, match="second run"):
                engine.step([StepEntry(s, t[3:], [0]) for s, t in zip(slots, seqs)])
            mixer.forward = real
            assert calls == [0, 2]                      # the first run had changed its state already
            for g, b in zip(engine.cache.state_groups.values(), before):
                assert torch.equal(g.data, b)
            assert [engine.cache.length(s) for s in slots] == [3, 3]
            engine.cache.check()
        return engine.step([StepEntry(s, t[3:], list(range(len(t) - 3))) for s, t in zip(slots, seqs)]).cpu()

    assert torch.equal(run(True), run(False))


@register("mixer", "toy_decay_on_the_gpu")
class ToyDecayOnTheGpu(ToyDecayMixer):
    """The same recurrence, but a step in which every sequence brings one token does GPU work only:
    the states of the step's slots are gathered, advanced and put back by index. So the part is
    graph_safe, and the engine runs such steps at the sizes of its ladder, records them and replays
    them. Rows of padding bring the cache's padding slot, whose state they advance and nobody
    reads; the part needs no word about them. Prompts take the host's loop."""
    graph_safe = True

    def forward(self, ctx, y, x):
        meta = ctx.meta
        if meta.max_new > 1:
            return super().forward(ctx, y, x)
        state = ctx.cache.state_views(ctx.cache_entry)[0]           # [slots + the padding slot, hidden]
        proj = (y.float()[:, None, :] * self.w[None]).sum(-1)
        slots = meta.slots.long()
        s = self.decay * state.index_select(0, slots) + proj
        state.index_copy_(0, slots, s)
        x += s


def test_a_graph_safe_mixer_with_state_through_padded_and_replayed_decode_steps():
    """Five sequences decode together (steps of six rows, one of them padding), then three of them go
    on (steps of three): first as they are, then recorded, then replayed. The logits are those of
    the mixer that loops on the host and is never recorded, and those of the sequences run whole;
    the padding slot's state is made NaN beforehand, so a row that read it would show."""
    import dataclasses
    spec = toy_spec()
    gpu_layer = dataclasses.replace(spec.layers[0], mixer=PartSpec("toy_decay_on_the_gpu", spec.layers[0].mixer.params))
    gpu_spec = dataclasses.replace(spec, layers=[gpu_layer, spec.layers[1]])
    from herbert_rs_amd.engine.model import Model
    from herbert_rs_amd.weights import random_tensors
    w = random_tensors(Model(spec).tensor_needs(), 3, "float32", std=0.15, norm_std=0.1)
    g = torch.Generator().manual_seed(5)
    lengths, more = [3, 9, 1, 6, 4], [20, 8, 20, 8, 20]
    seqs = [torch.randint(0, 60, (n + m,), generator=g).tolist() for n, m in zip(lengths, more)]

    def run(model_spec):
        engine = Engine(None, model_spec, w, dtype="float32", max_tokens=64 * 8)
        for group in engine.cache.state_groups.values():
            group.data[:, engine.cache.pad_slot] = float("nan")
        slots = [engine.alloc_slot() for _ in seqs]
        rows = [[] for _ in seqs]
        first = engine.step([StepEntry(s, t[:n], [n - 1]) for s, t, n in zip(slots, seqs, lengths)]).cpu()
        for i in range(len(seqs)):
            rows[i].append(first[i])
        for step in range(max(more)):
            live = [i for i in range(len(seqs)) if step < more[i]]
            out = engine.step([StepEntry(slots[i], [seqs[i][lengths[i] + step]], [0]) for i in live]).cpu()
            for r, i in enumerate(live):
                rows[i].append(out[r])
        return engine, [torch.stack(r) for r in rows]

    on_gpu, got = run(gpu_spec)
    on_host, want = run(spec)
    assert on_gpu.use_graphs and on_gpu.graphs_captured >= 2 and sorted(on_gpu._decode) == [3, 6]
    assert not on_host.use_graphs and on_host.graphs_captured == 0
    for a, b in zip(got, want):
        assert torch.isfinite(a).all() and torch.allclose(a, b, atol=1e-5)
    for i, t in enumerate(seqs):            # and the sequences whole, alone
        slot = on_host.alloc_slot()
        whole = on_host.step([StepEntry(slot, t, list(range(lengths[i] - 1, len(t))))]).cpu()
        on_host.free_slot(slot)
        assert torch.allclose(got[i], whole, atol=1e-4)


@register("mixer", "toy_counting_attention")
class ToyCountingAttention(Attention):
    """The library's attention with a state of fixed size beside its keys and values: how many
    tokens the sequence has brought so far. Its cache need is a pair, so the entry has pages in
    a group of keys and values and a number a slot in a group of state. GPU work only."""

    def cache_need(self):
        return (super().cache_need(), StateNeed((1,), torch.float32))

    def forward(self, ctx, y, x, **how):
        counts = ctx.cache.state_views(ctx.cache_entry)[0]          # [slots + the padding slot, 1]
        starts = ctx.meta.seq_starts
        counts.index_add_(0, ctx.meta.slots.long(), (starts[1:] - starts[:-1]).float()[:, None])
        super().forward(ctx, y, x, **how)


def test_a_mixer_whose_cache_need_is_keys_and_values_and_a_state():
    import dataclasses
    from herbert_rs_amd.errors import CacheError
    plain_spec = small_spec(2, [ScheduleEntry(0), ScheduleEntry(1)])
    counting = dataclasses.replace(plain_spec.layers[0], mixer=PartSpec("toy_counting_attention",
                                                                        plain_spec.layers[0].mixer.params))
    spec = dataclasses.replace(plain_spec, layers=[counting, plain_spec.layers[1]])
    w = weights_for(plain_spec, seed=11)
    g = torch.Generator().manual_seed(2)
    lengths, more = [7, 2, 70, 5, 1], [12, 12, 5, 12, 5]
    seqs = [torch.randint(0, 60, (n + m,), generator=g).tolist() for n, m in zip(lengths, more)]

    def run(model_spec):
        engine = Engine(None, model_spec, w, dtype="float32", max_tokens=64 * 8, max_slots=len(seqs))
        slots = [engine.alloc_slot() for _ in seqs]
        out = [engine.step([StepEntry(s, t[:n], [n - 1]) for s, t, n in zip(slots, seqs, lengths)]).cpu()]
        for step in range(max(more)):
            live = [i for i in range(len(seqs)) if step < more[i]]
            out.append(engine.step([StepEntry(slots[i], [seqs[i][lengths[i] + step]], [0]) for i in live]).cpu())
        return engine, slots, torch.cat(out)

    engine, slots, got = run(spec)
    _, _, want = run(plain_spec)
    assert torch.equal(got, want)                           # the attention itself is the library's
    assert engine.use_graphs and engine.graphs_captured >= 2
    needs = engine.model.cache_needs()
    assert isinstance(needs[0], tuple) and isinstance(needs[1], KVNeed)
    assert len(engine.cache.kv_groups) == 1 and len(engine.cache.state_groups) == 1     # both layers' pages in one group
    counts = engine.cache.state_views(0)[0][:, 0].cpu()
    assert [int(counts[s]) for s in slots] == [len(t) for t in seqs]
    with pytest.raises(CacheError, match="state"):
        engine.truncate(slots[0], 3)
    engine.free_slot(slots[2])
    again = engine.alloc_slot()
    assert again == slots[2] and float(engine.cache.state_views(0)[0][again, 0]) == 0.0
    engine.cache.check()


# ---- a toy feed-forward with routing and a toy position encoding, defined here
@register("feed_forward", "toy_routed")
class ToyRoutedFeedForward(Part):
    """Two experts; the router's larger logit (float32) picks one for each token:
    out = W2[e] relu(W1[e] y). The routing stays inside the part."""

    def __init__(self, hidden_size, intermediate_size, names, shared=None):
        self.h, self.i, self.names = hidden_size, intermediate_size, dict(names)

    def tensor_needs(self):
        n = self.names
        return {n["router"]: TensorNeed((2, self.h)), n["w1"]: TensorNeed((2 * self.i, self.h)),
                n["w2"]: TensorNeed((2 * self.h, self.i))}

    def load(self, tensors, rt):
        n = self.names
        self.router = tensors[n["router"]].to(rt.device).float()
        self.w1 = tensors[n["w1"]].to(rt.device).float().view(2, self.i, self.h)
        self.w2 = tensors[n["w2"]].to(rt.device).float().view(2, self.h, self.i)

    def forward(self, ctx, y, x):
        y = y.float()
        expert = (y @ self.router.T).argmax(-1)
        for e in range(2):
            rows = (expert == e).nonzero().flatten()
            if len(rows):
                x[rows] += torch.relu(y[rows] @ self.w1[e].T) @ self.w2[e].T


@register("position", "toy_slow_rope")
class ToySlowRope(Part):
    """Half-split rotation of the first `rotary_dims` of a head by angles of position / 4: another
    table behind the hook the attention part asks (`rotation()`)."""
    graph_safe = True

    def __init__(self, rotary_dims, max_positions):
        self.rotary_dims, self.max_positions = rotary_dims, max_positions

    def angles(self):
        inv_freq = 1.0 / (100.0 ** (2.0 * torch.arange(self.rotary_dims // 2, dtype=torch.float32) / self.rotary_dims))
        return (torch.arange(self.max_positions, dtype=torch.float32) / 4.0)[:, None] * inv_freq[None]

    def load(self, tensors, rt):
        a = self.angles()
        self.cos, self.sin = torch.cos(a).contiguous().to(rt.device), torch.sin(a).contiguous().to(rt.device)

    def rotation(self):
        return self.cos, self.sin, self.rotary_dims


def test_toy_routed_feed_forward_and_toy_position_encoding():
    hidden, inter = 40, 24
    pos = PartSpec("toy_slow_rope", {"rotary_dims": 8, "max_positions": 256})
    names = {k: "L." + k for k in ("q", "k", "v", "o", "q_norm", "k_norm")}
    layer = LayerSpec(PartSpec("prenorm"),
                      PartSpec("attention", dict(hidden_size=hidden, num_heads=4, num_kv_heads=2, head_dim=16, eps=1e-6,
                                                 position=pos, names=names)),
                      PartSpec("toy_routed", {"hidden_size": hidden, "intermediate_size": inter,
                                              "names": {"router": "L.r", "w1": "L.w1", "w2": "L.w2"}}),
                      {"input": PartSpec("rmsnorm", {"size": hidden, "eps": 1e-6, "weight": "L.n1"}),
                       "post_mixer": PartSpec("rmsnorm", {"size": hidden, "eps": 1e-6, "weight": "L.n2"})})
    base = small_spec(1, [ScheduleEntry(0)])
    spec = ModelSpec(hidden_size=hidden, vocab_size=60, max_positions=256, embedding=base.embedding, layers=[layer],
                     schedule=[ScheduleEntry(0), ScheduleEntry(0)], final_norm=base.final_norm, head=base.head)
    w = weights_for(spec, seed=6)
    tokens = [5, 9, 33, 2, 41, 17, 8, 11, 3, 50, 27]
    positions = list(range(len(tokens)))
    table = ToySlowRope(8, 256).angles()

    def rotate(u):          # [T, heads, 16]: the first 8 of a head, pairs (j, j + 4)
        c, s = torch.cos(table[positions])[:, None, :], torch.sin(table[positions])[:, None, :]
        a, b = u[..., :4], u[..., 4:8]
        return torch.cat([a * c - b * s, a * s + b * c, u[..., 8:]], -1)

    x = pops.embedding(tokens, w["emb"])
    picked = []
    for _ in range(2):
        y = pops.rms_norm(x, w["L.n1"], 1e-6)
        q = rotate(pops.head_rms_norm(pops.split_heads(pops.linear(y, w["L.q"]), 4, 16), w["L.q_norm"], 1e-6))
        k = rotate(pops.head_rms_norm(pops.split_heads(pops.linear(y, w["L.k"]), 2, 16), w["L.k_norm"], 1e-6))
        v = pops.split_heads(pops.linear(y, w["L.v"]), 2, 16)
        x = x + pops.linear(pops.causal_attention(q, k, v, positions).reshape(len(tokens), 64), w["L.o"])
        y = pops.rms_norm(x, w["L.n2"], 1e-6)
        expert = (y @ w["L.r"].T).argmax(-1)
        picked += expert.tolist()
        w1, w2 = w["L.w1"].view(2, inter, hidden), w["L.w2"].view(2, hidden, inter)
        x = x + torch.stack([torch.relu(y[t] @ w1[e].T) @ w2[e].T for t, e in enumerate(expert.tolist())])
    assert 0 < sum(picked) < len(picked)                    # both experts are in use
    want = pops.linear(pops.rms_norm(x, w["fn"], 1e-6), w["emb"])
    assert torch.allclose(run_engine(spec, w, tokens), want, atol=1e-4)
    assert torch.allclose(run_engine(spec, w, tokens, cut=4), want, atol=1e-4)


def _small_positions(shape, gen, device, std, norm_std):
    return 0.3 * torch.randn(shape, generator=gen, dtype=torch.float32, device=device)


@register("embedding", "toy_table_with_learned_positions")
class ToyLearnedPositions(Part):
    """A position encoding that is no rotation: a learned row for every position, added to the
    token's embedding (the mixers then take the position "none"). It is an embedding part of its
    own: what it needs of the step, each token's absolute position, is in ctx.meta. Its table is
    a tensor of a kind the library does not know and brings its own random initialiser."""
    graph_safe = True

    def __init__(self, vocab_size, hidden_size, max_positions, weight, positions_weight, shared=None):
        from herbert_rs_amd.parts.io import TokenEmbedding
        self.tokens = TokenEmbedding(vocab_size, hidden_size, weight)
        self.max_positions, self.hidden_size, self.positions_name = max_positions, hidden_size, positions_weight

    def tensor_needs(self):
        needs = dict(self.tokens.tensor_needs())
        needs[self.positions_name] = TensorNeed((self.max_positions, self.hidden_size), "learned_positions",
                                                init=_small_positions)
        return needs

    def load(self, tensors, rt, shared_with_head=False):
        self.tokens.load(tensors, rt, shared_with_head=shared_with_head)
        self.linear = self.tokens.linear           # what a tied head multiplies with
        self.rows = tensors[self.positions_name].to(rt.device).float()

    def forward(self, ctx, token_ids):
        x = self.tokens.forward(ctx, token_ids)
        x += self.rows[ctx.meta.positions.long()]
        return x


def test_toy_position_encoding_that_is_no_rotation():
    base = small_spec(2, [ScheduleEntry(0), ScheduleEntry(1)], rope=False)
    emb = PartSpec("toy_table_with_learned_positions",
                   {"vocab_size": 60, "hidden_size": 40, "max_positions": 256, "weight": "emb", "positions_weight": "pos"})
    spec = ModelSpec(hidden_size=40, vocab_size=60, max_positions=256, embedding=emb, layers=base.layers,
                     schedule=base.schedule, final_norm=base.final_norm, head=base.head)
    w = weights_for(spec, seed=9)
    assert tuple(w["pos"].shape) == (256, 40) and 0.2 < float(w["pos"].std()) < 0.4
    tokens = [5, 9, 33, 2, 41, 17, 8, 11, 3]
    positions = list(range(len(tokens)))
    x = pops.embedding(tokens, w["emb"]) + w["pos"][positions]
    for p in ("L0.", "L1."):
        x, _ = plain_layer(w, p, x, positions, rope=False)
    want = pops.linear(pops.rms_norm(x, w["fn"], 1e-6), w["emb"])
    assert torch.allclose(run_engine(spec, w, tokens), want, atol=1e-4)
    assert torch.allclose(run_engine(spec, w, tokens, cut=4), want, atol=1e-4)      # positions go on from the cache's length
    # In one layer without rotation the last token sees the set of earlier tokens, not their order:
    # its logits stay when two earlier tokens change places. With the learned rows they move.
    swapped = [9, 5] + tokens[2:]
    one = small_spec(1, [ScheduleEntry(0)], rope=False)
    w1 = weights_for(one, seed=9)
    assert torch.allclose(run_engine(one, w1, swapped)[-1], run_engine(one, w1, tokens)[-1], atol=1e-4)
    toy_one = ModelSpec(hidden_size=40, vocab_size=60, max_positions=256, embedding=emb, layers=one.layers,
                        schedule=one.schedule, final_norm=one.final_norm, head=one.head)
    w3 = weights_for(toy_one, seed=9)
    assert not torch.allclose(run_engine(toy_one, w3, swapped)[-1], run_engine(toy_one, w3, tokens)[-1], atol=1e-3)


# ---- a toy arrangement of a layer and a toy norm, between the library's own blocks
@register("norm", "toy_centred_norm")
class ToyCentredNorm(Part):
    """y = (x - mean) / sqrt(var + eps) * w: not of the form x * w / rms(x), so no product can
    finish it; it has its own (library) arithmetic and knows nothing of norms handed on."""

    def __init__(self, size, eps, weight):
        self.size, self.eps, self.weight_name = size, eps, weight

    def tensor_needs(self):
        return {self.weight_name: TensorNeed((self.size,), "scale")}

    def load(self, tensors, rt):
        self.w = tensors[self.weight_name].to(rt.device).float()
        self.dtype = rt.dtype

    def forward(self, ctx, x, rows=None, name="normed"):
        x = x.float() if rows is None else x.float()[rows.long()]
        c = x - x.mean(-1, keepdim=True)
        return (c / torch.sqrt((c * c).mean(-1, keepdim=True) + self.eps) * self.w).to(self.dtype)


@register("block", "toy_parallel")
class ToyParallelBlock(Part):
    """x += mixer(norm(x)) + feed_forward(norm(x)): both parts read the same normed rows."""

    def __init__(self, mixer, feed_forward, norms):
        self.mixer, self.feed_forward, self.norm = mixer, feed_forward, norms["input"]

    def parts(self):
        return [self.norm, self.mixer, self.feed_forward]

    def forward(self, ctx, x):
        y = self.norm.forward(ctx, x).clone()
        self.mixer.forward(ctx, y, x)
        self.feed_forward.forward(ctx, y, x)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_toy_block_and_toy_norm_between_the_library_s_blocks(dtype):
    from .bounds import close
    hidden, inter, vocab = 64, 96, 90
    pos = PartSpec("rope", {"theta": 1e4, "rotary_dims": 16, "max_positions": 256})

    def layer(i, block, norms):
        p = f"L{i}."
        names = {k: p + k for k in ("q", "k", "v", "o", "q_norm", "k_norm")}
        return LayerSpec(PartSpec(block),
                         PartSpec("attention", dict(hidden_size=hidden, num_heads=4, num_kv_heads=2, head_dim=16,
                                                    eps=1e-6, position=pos, names=names)),
                         PartSpec("swiglu", {"hidden_size": hidden, "intermediate_size": inter,
                                             "names": {"gate": p + "g", "up": p + "u", "down": p + "d"}}), norms)

    def rms(i, k):
        return PartSpec("rmsnorm", {"size": hidden, "eps": 1e-6, "weight": f"L{i}.{k}"})

    layers = [layer(0, "prenorm", {"input": rms(0, "n1"), "post_mixer": rms(0, "n2")}),
              layer(1, "toy_parallel", {"input": PartSpec("toy_centred_norm", {"size": hidden, "eps": 1e-3,
                                                                               "weight": "L1.n1"})}),
              layer(2, "prenorm", {"input": rms(2, "n1"), "post_mixer": rms(2, "n2")})]
    spec = ModelSpec(hidden_size=hidden, vocab_size=vocab, max_positions=256,
                     embedding=PartSpec("table", {"vocab_size": vocab, "hidden_size": hidden, "weight": "emb"}),
                     layers=layers, schedule=[ScheduleEntry(0), ScheduleEntry(1), ScheduleEntry(2)],
                     final_norm=rms(3, "fn"),
                     head=PartSpec("linear", {"vocab_size": vocab, "hidden_size": hidden, "weight": "head",
                                              "tied_to_embedding": True}))
    # (weights of the tiny configurations' scale, whose bounds are used below; matrices that
    # bfloat16 holds exactly, so that both dtypes run the same model)
    from herbert_rs_amd.engine.model import Model
    from herbert_rs_amd.weights import random_tensors
    w = random_tensors(Model(spec).tensor_needs(), 12, "float32", std=0.05, norm_std=0.1)
    w = {k: v.to(torch.bfloat16).float() if v.dim() == 2 else v for k, v in w.items()}
    tokens = [5, 9, 33, 2, 41, 17, 8, 11, 3, 50, 27, 64, 80, 1]
    positions = list(range(len(tokens)))

    x = pops.embedding(tokens, w["emb"])
    x, _ = plain_layer_of(w, "L0.", x, positions, inter)
    c = x - x.mean(-1, keepdim=True)
    y = c / torch.sqrt((c * c).mean(-1, keepdim=True) + 1e-3) * w["L1.n1"]
    x = x + plain_mixer(w, "L1.", y, positions) + pops.swiglu_mlp(y, w["L1.g"], w["L1.u"], w["L1.d"])
    x, _ = plain_layer_of(w, "L2.", x, positions, inter)
    want = pops.linear(pops.rms_norm(x, w["L3.fn"], 1e-6), w["emb"]).numpy()

    engine = Engine(None, spec, w, dtype=dtype, max_tokens=256)
    for cut in (len(tokens), 6):             # whole, then a prompt of 6 and one token at a time
        s = engine.alloc_slot()
        got = [engine.step([StepEntry(s, tokens[:cut], list(range(cut)))]).cpu()]
        got += [engine.step([StepEntry(s, [t], [0])]).cpu() for t in tokens[cut:]]
        engine.free_slot(s)
        got = torch.cat(got).numpy()
        for t in positions:
            ok, err = close(got[t], want[t], dtype, "A", f"toy block cut {cut}")
            assert ok, (cut, t, err)


def plain_mixer(w, p, y, positions):
    q = pops.apply_rope(pops.head_rms_norm(pops.split_heads(pops.linear(y, w[p + "q"]), 4, 16), w[p + "q_norm"], 1e-6),
                        positions, 1e4)
    k = pops.apply_rope(pops.head_rms_norm(pops.split_heads(pops.linear(y, w[p + "k"]), 2, 16), w[p + "k_norm"], 1e-6),
                        positions, 1e4)
    v = pops.split_heads(pops.linear(y, w[p + "v"]), 2, 16)
    return pops.linear(pops.causal_attention(q, k, v, positions).reshape(len(positions), 64), w[p + "o"])


def plain_layer_of(w, p, x, positions, inter):
    x = x + plain_mixer(w, p, pops.rms_norm(x, w[p + "n1"], 1e-6), positions)
    y = pops.rms_norm(x, w[p + "n2"], 1e-6)
    return x + pops.swiglu_mlp(y, w[p + "g"], w[p + "u"], w[p + "d"]), None
