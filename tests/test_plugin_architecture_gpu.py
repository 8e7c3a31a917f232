"""A whole architecture defined outside the framework's files: a module (written here into a
temporary folder) with a feed-forward of its own, a configuration class with its own config.json
keys, a spec builder and a registry entry. Named in HERBERT_PLUGINS it is known to the programs:
a model folder with random weights is written for it, `bin/trace_run` replays a trace on it in a
process of its own (whole prompts, then one token at a time, unequal lengths), and the logits are
those of the formulas written out here with the plain implementation's parts."""
import json
import os
import subprocess
import sys
import textwrap

import numpy as np
import pytest
import torch

from .plain import ops as pops

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))

MODULE = textwrap.dedent('''
    """A toy family: pre-norm layers of the library's attention (no q/k norm, rotation of half a
    head) and a feed-forward of its own, down(relu(up(y))^2); names of its own throughout."""
    from dataclasses import asdict, dataclass

    import torch

    from herbert_rs_amd.config import ChatFormat, register_architecture
    from herbert_rs_amd.parts import LayerSpec, ModelSpec, Part, PartSpec, ScheduleEntry, register
    from herbert_rs_amd.weights import TensorNeed
    from herbert_rs_amd.weights.names import NameMap


    @register("feed_forward", "toy_relu_squared")
    class ReluSquared(Part):
        def __init__(self, width, inner, names, shared=None):
            self.width, self.inner, self.names = width, inner, dict(names)

        def tensor_needs(self):
            return {self.names["up"]: TensorNeed((self.inner, self.width)),
                    self.names["down"]: TensorNeed((self.width, self.inner))}

        def load(self, tensors, rt):
            self.up = tensors[self.names["up"]].to(rt.device).float()
            self.down = tensors[self.names["down"]].to(rt.device).float()

        def forward(self, ctx, y, x):
            x += (torch.relu(y.float() @ self.up.T) ** 2) @ self.down.T


    @dataclass(frozen=True)
    class ToyConfig:
        n_layer: int
        d_model: int
        n_head: int
        n_kv: int
        d_head: int
        d_ff: int
        n_vocab: int
        n_ctx: int
        eps: float
        base: float

        @classmethod
        def from_dict(cls, raw):
            return cls(**{k: raw[k] for k in cls.__dataclass_fields__})

        def to_dict(self):
            return dict(asdict(self), architectures=["ToyFamilyLM"])


    def build_spec(c):
        position = PartSpec("rope", {"theta": c.base, "rotary_dims": c.d_head // 2, "max_positions": c.n_ctx,
                                     "scaling": None})
        layers = []
        for i in range(c.n_layer):
            p = f"h.{i}."
            layers.append(LayerSpec(
                PartSpec("prenorm"),
                PartSpec("attention", {"hidden_size": c.d_model, "num_heads": c.n_head, "num_kv_heads": c.n_kv,
                                       "head_dim": c.d_head, "eps": c.eps, "qk_norm": False, "window": None,
                                       "position": position,
                                       "names": {"q": p + "q", "k": p + "k", "v": p + "v", "o": p + "o"}}),
                PartSpec("toy_relu_squared", {"width": c.d_model, "inner": c.d_ff,
                                              "names": {"up": p + "up", "down": p + "down"}}),
                {"input": PartSpec("rmsnorm", {"size": c.d_model, "eps": c.eps, "weight": p + "n1"}),
                 "post_mixer": PartSpec("rmsnorm", {"size": c.d_model, "eps": c.eps, "weight": p + "n2"})}))
        return ModelSpec(hidden_size=c.d_model, vocab_size=c.n_vocab, max_positions=c.n_ctx,
                         embedding=PartSpec("table", {"vocab_size": c.n_vocab, "hidden_size": c.d_model, "weight": "wte"}),
                         layers=layers, schedule=[ScheduleEntry(i) for i in range(c.n_layer)],
                         final_norm=PartSpec("rmsnorm", {"size": c.d_model, "eps": c.eps, "weight": "nf"}),
                         head=PartSpec("linear", {"vocab_size": c.n_vocab, "hidden_size": c.d_model, "weight": "head",
                                                  "tied_to_embedding": False}),
                         eos_token_id=None)


    register_architecture("ToyFamilyLM", ToyConfig, build_spec, model_types=("toy_family",),
                          name_map=NameMap(prefixes=(("toy.", ""),), layer_prefix="h.", layer_aliases={}, fused={}),
                          chat=ChatFormat(lambda user, system=None: user))
''')

RAW = dict(architectures=["ToyFamilyLM"], n_layer=2, d_model=48, n_head=6, n_kv=2, d_head=16, d_ff=80, n_vocab=90,
           n_ctx=256, eps=1e-5, base=10000.0)


def plain_logits(w, tokens):
    """The toy family's formulas with the plain implementation's parts: whole sequence, no cache."""
    c = RAW
    positions = list(range(len(tokens)))
    half = c["d_head"] // 2
    inv_freq = 1.0 / (c["base"] ** (2.0 * torch.arange(half // 2, dtype=torch.float32) / half))
    angles = torch.tensor(positions, dtype=torch.float32)[:, None] * inv_freq[None]
    cos, sin = torch.cos(angles)[:, None, :], torch.sin(angles)[:, None, :]

    def rotate(u):          # the first half of a head, pairs (j, j + half / 2)
        a, b = u[..., :half // 2], u[..., half // 2:half]
        return torch.cat([a * cos - b * sin, a * sin + b * cos, u[..., half:]], -1)

    x = pops.embedding(tokens, w["wte"])
    for i in range(c["n_layer"]):
        p = f"h.{i}."
        y = pops.rms_norm(x, w[p + "n1"], c["eps"])
        q = rotate(pops.split_heads(pops.linear(y, w[p + "q"]), c["n_head"], c["d_head"]))
        k = rotate(pops.split_heads(pops.linear(y, w[p + "k"]), c["n_kv"], c["d_head"]))
        v = pops.split_heads(pops.linear(y, w[p + "v"]), c["n_kv"], c["d_head"])
        x = x + pops.linear(pops.causal_attention(q, k, v, positions).reshape(len(tokens), -1), w[p + "o"])
        y = pops.rms_norm(x, w[p + "n2"], c["eps"])
        x = x + pops.linear(torch.relu(pops.linear(y, w[p + "up"])) ** 2, w[p + "down"])
    return pops.linear(pops.rms_norm(x, w["nf"], c["eps"]), w["head"])


def test_an_architecture_of_a_plugin_runs_through_the_replay_program(tmp_path):
    from safetensors.torch import load_file
    (tmp_path / "toy_family.py").write_text(MODULE)
    env = dict(os.environ, HERBERT_PLUGINS="toy_family",
               PYTHONPATH=os.pathsep.join([str(tmp_path), ROOT, os.environ.get("PYTHONPATH", "")]))
    folder = tmp_path / "model"
    # the folder is written by the framework's own random-weights mode, in a process that knows the plugin
    made = subprocess.run([sys.executable, "-c", "import sys, json, herbert_rs_amd as hb; "
                           "hb.write_random_model(sys.argv[1], json.loads(sys.argv[2]), seed=4, dtype='float32', "
                           "std=0.08, norm_std=0.1)", str(folder), json.dumps(RAW)],
                          env=env, capture_output=True, text=True, timeout=240)
    assert made.returncode == 0, made.stderr
    assert json.loads((folder / "config.json").read_text())["n_layer"] == 2
    w = {k: v.float() for k, v in load_file(str(folder / "model.safetensors")).items()}
    assert set(w) == {"wte", "nf", "head"} | {f"h.{i}.{n}" for i in range(2) for n in ("q", "k", "v", "o", "up", "down", "n1", "n2")}
    g = torch.Generator().manual_seed(9)
    seqs = {"a": torch.randint(0, 90, (70,), generator=g).tolist(), "b": torch.randint(0, 90, (9,), generator=g).tolist()}
    first = {"a": 66, "b": 5}
    steps = [{"step": 0, "entries": [{"id": r, "tokens": seqs[r][:first[r]], "want": list(range(first[r]))} for r in seqs],
              "end": []}]
    for j in range(4):
        steps.append({"step": j + 1, "entries": [{"id": r, "tokens": [seqs[r][first[r] + j]], "want": [0]} for r in seqs],
                      "end": ["a", "b"] if j == 3 else []})
    out = tmp_path / "out"
    run = subprocess.run([os.path.join(ROOT, "bin", "trace_run"), "--model", str(folder), "--dtype", "float32",
                          "--out", str(out), "--max-tokens", "256"],
                         input="\n".join(json.dumps(s) for s in steps) + "\n", env=env, capture_output=True, text=True,
                         timeout=300)
    assert run.returncode == 0, run.stderr
    assert [l for l in run.stdout.split("\n") if l.startswith("done")] == [f"done {j}" for j in range(5)]
    ref = {r: plain_logits(w, seqs[r][:first[r] + 4]).numpy() for r in seqs}
    got0 = np.fromfile(out / "0.f32", dtype="<f4").reshape(-1, 90)
    assert np.abs(got0[:66] - ref["a"][:66]).max() < 1e-4 and np.abs(got0[66:] - ref["b"][:5]).max() < 1e-4
    for j in range(4):
        got = np.fromfile(out / f"{j + 1}.f32", dtype="<f4").reshape(2, 90)
        assert np.abs(got[0] - ref["a"][66 + j]).max() < 1e-4 and np.abs(got[1] - ref["b"][5 + j]).max() < 1e-4
    # without the plugin the architecture is unknown, and the error names those that are known
    bare = dict(env)
    del bare["HERBERT_PLUGINS"]
    run = subprocess.run([os.path.join(ROOT, "bin", "trace_run"), "--model", str(folder), "--dtype", "float32",
                          "--out", str(out), "--max-tokens", "256"], input="", env=bare, capture_output=True, text=True,
                         timeout=120)
    assert run.returncode == 1 and "unknown architecture 'ToyFamilyLM'" in run.stderr and "Qwen3ForCausalLM" in run.stderr
