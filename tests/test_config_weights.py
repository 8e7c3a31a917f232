"""Configuration (keys, defaults, errors, registry) and weights (reading, errors, random folders)."""
import json
import os

import numpy as np
import pytest
import torch
from safetensors.torch import load_file, save_file

from herbert_rs_amd.config import Qwen3Config, load_config, registered_architectures
from herbert_rs_amd.config.registry import resolve_architecture
from herbert_rs_amd.engine.model import Model
from herbert_rs_amd.errors import ConfigError, ModelLoadError
from herbert_rs_amd.weights import read_tensors
from herbert_rs_amd.weights.bf16 import bf16_bits_to_f32, f32_to_bf16_bits

from .tiny import TINY_A, TINY_B, TINY_C, make_folder, spec_of


def minimal(**over):
    raw = dict(vocab_size=100, hidden_size=32, num_hidden_layers=2, num_attention_heads=4,
               num_key_value_heads=2, intermediate_size=64, max_position_embeddings=64,
               rope_theta=10000.0)
    raw.update(over)
    return {k: v for k, v in raw.items() if v is not ...}


def test_defaults_of_the_reference():
    cfg = Qwen3Config.from_dict(minimal())
    assert cfg.rms_norm_eps == 1e-5                 # crates/core/src/config.rs:583-585
    assert cfg.tie_word_embeddings is True          # :199-202
    assert cfg.head_dim == 8                        # hidden / heads, :496-498
    assert cfg.eos_token_id == 151643               # :283-287
    assert cfg.layer_windows == (None, None)
    assert (cfg.q_dim, cfg.kv_dim, cfg.num_kv_groups) == (32, 16, 2)


def test_decoupled_head_dim_and_eos_forms():
    cfg = Qwen3Config.from_dict(minimal(head_dim=16, eos_token_id=[7, 9]))
    assert cfg.q_dim == 64 and cfg.eos_token_id == 7
    assert Qwen3Config.from_dict(minimal(eos_token_id=5)).eos_token_id == 5
    nested = minimal(rope_theta=..., rope_parameters={"rope_theta": 5e5, "rope_type": "default"})
    assert Qwen3Config.from_dict(nested).rope_theta == 5e5


@pytest.mark.parametrize("over,word", [
    (dict(rope_theta=...), "rope_theta"),
    (dict(vocab_size=...), "vocab_size"),
    (dict(num_key_value_heads=3), "divisible"),
    (dict(head_dim=7), "even"),
    (dict(hidden_size=0), "hidden_size"),
    (dict(num_hidden_layers=0), "num_layers"),
    (dict(intermediate_size=0), "intermediate_size"),
    (dict(rms_norm_eps=0.0), "rms_norm_eps"),
    (dict(rope_theta=-1.0), "rope_theta"),
    (dict(max_position_embeddings=0), "max_position_embeddings"),
    (dict(num_experts=8), "expert"),
    (dict(rope_scaling={"type": "llama3", "factor": 4.0}), "llama3"),
    (dict(rope_scaling={"type": "yarn", "factor": 4.0, "beta_fast": 2.0, "beta_slow": 2.0}), "beta_fast"),
    (dict(text_config={}), "text_config"),
    (dict(layer_types=["full_attention"]), "layer_types"),
    (dict(layer_types=["sliding_attention", "full_attention"]), "sliding_window"),
    (dict(vocab_size="many"), "integer"),
    (dict(partial_rotary_factor=1.5), "partial_rotary_factor"),
    (dict(partial_rotary_factor=0.1), "partial_rotary_factor"),          # 1.6 of 16 dimensions: cut to 1
])
def test_config_errors_name_the_key(over, word):
    with pytest.raises(ConfigError, match=word):
        Qwen3Config.from_dict(minimal(**over))


def test_partial_rotation_as_the_reference_derives_it():
    """crates/core/src/config.rs:516-525: top level, else rope_parameters; float32 product cut to an integer."""
    assert Qwen3Config.from_dict(TINY_A).rotary_dims == 16
    assert Qwen3Config.from_dict(dict(TINY_A, partial_rotary_factor=0.5)).rotary_dims == 8
    nested = dict(TINY_B, rope_parameters={"partial_rotary_factor": 0.25, "rope_theta": 5.0})
    cfg = Qwen3Config.from_dict(nested)
    assert cfg.rotary_dims == 8 and cfg.rope_theta == 1000000.0          # the top-level theta wins
    assert Qwen3Config.from_dict(cfg.to_dict()) == cfg
    from herbert_rs_amd.models.qwen3 import build_spec
    assert build_spec(cfg).layers[0].mixer.params["position"].params["rotary_dims"] == 8


def test_rope_scaling_as_the_reference_reads_it():
    """crates/core/src/config.rs:547-580."""
    plain = Qwen3Config.from_dict(TINY_A)
    assert plain.rope_scaling[0] == "default"
    assert Qwen3Config.from_dict(dict(TINY_A, rope_scaling={"type": "linear", "factor": 1.0})).rope_scaling[0] == "default"
    lin = Qwen3Config.from_dict(dict(TINY_A, rope_scaling={"type": "linear", "factor": 2.5}))
    assert lin.rope_scaling[:2] == ("linear", 2.5)
    yarn = Qwen3Config.from_dict(dict(TINY_A, rope_scaling={"rope_type": "yarn", "factor": 4.0,
                                                             "original_max_position_embeddings": 32}))
    assert yarn.rope_scaling == ("yarn", 4.0, 32, 32.0, 1.0)
    nested = Qwen3Config.from_dict(dict(TINY_A, rope_parameters={"rope_type": "yarn", "factor": 2.0, "beta_slow": 2.0},
                                        rope_scaling={"type": "linear", "factor": 8.0}))
    assert nested.rope_scaling == ("yarn", 2.0, None, 32.0, 2.0)          # rope_parameters wins
    for cfg in (lin, yarn, nested):
        assert Qwen3Config.from_dict(cfg.to_dict()) == cfg


def test_windows_from_both_forms():
    cfg = Qwen3Config.from_dict(minimal(sliding_window=16, layer_types=["sliding_attention", "full_attention"]))
    assert cfg.layer_windows == (16, None)
    cfg = Qwen3Config.from_dict(minimal(sliding_window=16, use_sliding_window=True, max_window_layers=1))
    assert cfg.layer_windows == (None, 16)
    cfg = Qwen3Config.from_dict(minimal(sliding_window=16, use_sliding_window=False))
    assert cfg.layer_windows == (None, None)
    assert Qwen3Config.from_dict(cfg.to_dict()) == cfg
    win = Qwen3Config.from_dict(TINY_C)
    assert Qwen3Config.from_dict(win.to_dict()) == win


def test_registry_by_architecture_and_model_type(tmp_path):
    assert "Qwen3ForCausalLM" in registered_architectures()
    assert resolve_architecture({"architectures": ["Qwen3ForCausalLM"]}).name == "Qwen3ForCausalLM"
    assert resolve_architecture({"model_type": "qwen3"}).name == "Qwen3ForCausalLM"
    assert resolve_architecture({}).name == "Qwen3ForCausalLM"        # model_type defaults to qwen3
    with pytest.raises(ConfigError, match="Qwen3ForCausalLM"):
        resolve_architecture({"architectures": ["LlamaForCausalLM"]})
    with pytest.raises(ConfigError, match="gpt2"):
        resolve_architecture({"model_type": "gpt2"})
    with open(tmp_path / "config.json", "w") as f:
        json.dump(TINY_B, f)
    arch, cfg = load_config(str(tmp_path))
    assert cfg.num_hidden_layers == 3 and cfg.eos_token_id == 383
    with pytest.raises(ConfigError, match="config.json"):
        load_config(str(tmp_path / "nothing"))


def test_the_tiny_configurations_differ_everywhere():
    a, b, c = (Qwen3Config.from_dict(t) for t in (TINY_A, TINY_B, TINY_C))
    for field in ("vocab_size", "hidden_size", "num_attention_heads", "head_dim", "intermediate_size",
                  "max_position_embeddings", "rope_theta", "rms_norm_eps", "num_kv_groups"):
        assert len({getattr(a, field), getattr(b, field), getattr(c, field)}) == 3, field
    assert a.tie_word_embeddings != b.tie_word_embeddings
    assert a.num_hidden_layers != b.num_hidden_layers
    assert c.layer_windows != a.layer_windows


# ---- weights
def needs_of(raw):
    return Model(spec_of(raw)[1]).tensor_needs()


def test_random_folder_reads_back(model_root):
    for dtype, tdt in (("float32", torch.float32), ("bfloat16", torch.bfloat16)):
        folder = make_folder(model_root, "B", dtype)
        needs = needs_of(TINY_B)
        tensors = read_tensors(folder, needs)
        assert set(tensors) == set(needs)
        assert "lm_head.weight" in needs and "lm_head.weight" not in needs_of(TINY_A)
        for name, t in tensors.items():
            assert tuple(t.shape) == tuple(needs[name].shape) and t.dtype == tdt     # kept as stored
        q = tensors["model.layers.0.self_attn.q_proj.weight"].float()
        assert tuple(q.shape) == (192, 96) and 0.04 < float(q.std()) < 0.06
        n = tensors["model.norm.weight"].float()
        assert abs(float(n.mean()) - 1.0) < 0.1 and float(n.std()) > 0.01
    again = make_folder(str(model_root) + "_again", "B", "float32")
    same = load_file(os.path.join(again, "model.safetensors"))
    first = load_file(os.path.join(make_folder(model_root, "B", "float32"), "model.safetensors"))
    assert all(torch.equal(same[k], first[k]) for k in first)          # the seed decides


def test_one_error_lists_missing_unexpected_and_wrong(model_root, tmp_path):
    src = make_folder(model_root, "A", "float32")
    tensors = load_file(os.path.join(src, "model.safetensors"))
    del tensors["model.layers.1.self_attn.q_norm.weight"]
    del tensors["model.norm.weight"]
    tensors["model.layers.0.mlp.gate_proj.weight"] = torch.zeros(128, 63)
    tensors["model.layers.0.self_attn.rotary_emb.inv_freq"] = torch.zeros(8)
    save_file(tensors, str(tmp_path / "model.safetensors"))
    with open(tmp_path / "config.json", "w") as f:
        json.dump(TINY_A, f)
    with pytest.raises(ModelLoadError) as err:
        read_tensors(str(tmp_path), needs_of(TINY_A), strict=True)
    text = str(err.value)
    assert "missing (2)" in text and "model.layers.1.self_attn.q_norm.weight" in text
    assert "model.norm.weight" in text
    assert "unexpected (1)" in text and "rotary_emb.inv_freq" in text
    assert "gate_proj.weight: expected [128, 64], got [128, 63]" in text
    # without `strict` the stray tensor is no fault, the others still are, in one error
    with pytest.raises(ModelLoadError) as err:
        read_tensors(str(tmp_path), needs_of(TINY_A))
    text = str(err.value)
    assert "missing (2)" in text and "expected [128, 64], got [128, 63]" in text
    assert "unexpected" not in text and "inv_freq" not in text


def test_unknown_names_are_passed_over_and_an_untied_model_needs_its_head(model_root, tmp_path):
    """Tensors nobody asks for are ignored as the reference ignores them
    (crates/backends/backend_common/src/loader_common.rs:679-685,1588): rotary buffers, and a
    stored head beside tied embeddings, which the reference drops for the embedding
    (loader_common.rs:1851-1872)."""
    src = make_folder(model_root, "A", "float32")
    plain = load_file(os.path.join(src, "model.safetensors"))
    tensors = dict(plain)
    tensors["lm_head.weight"] = torch.full((256, 64), 9.0)
    tensors["model.layers.0.self_attn.rotary_emb.inv_freq"] = torch.zeros(8)
    tensors["model.layers.1.self_attn.rotary_emb.inv_freq"] = torch.zeros(8)
    save_file(tensors, str(tmp_path / "model.safetensors"))
    ignored = []
    got = read_tensors(str(tmp_path), needs_of(TINY_A), ignored=ignored)
    assert set(got) == set(plain) and all(torch.equal(got[k], plain[k]) for k in plain)
    assert sorted(ignored) == ["lm_head.weight", "model.layers.0.self_attn.rotary_emb.inv_freq",
                               "model.layers.1.self_attn.rotary_emb.inv_freq"]
    with pytest.raises(ModelLoadError, match=r"unexpected \(3\)"):
        read_tensors(str(tmp_path), needs_of(TINY_A), strict=True)
    with pytest.raises(ModelLoadError, match="lm_head.weight"):
        read_tensors(src, needs_of(dict(TINY_A, tie_word_embeddings=False)))


def test_stored_dtypes_and_shards(tmp_path):
    from herbert_rs_amd.weights import TensorNeed
    save_file({"a": torch.ones(2, 2, dtype=torch.float16), "i": torch.arange(3, dtype=torch.int64)},
              str(tmp_path / "part1.safetensors"))
    save_file({"b": torch.ones(2, dtype=torch.float32)}, str(tmp_path / "part2.safetensors"))
    with open(tmp_path / "model.safetensors.index.json", "w") as f:
        json.dump({"weight_map": {"a": "part1.safetensors", "i": "x/part1.safetensors",
                                  "b": "part2.safetensors"}}, f)
    got = read_tensors(str(tmp_path), {"a": TensorNeed((2, 2)), "b": TensorNeed((2,), "scale"),
                                       "i": TensorNeed((3,), "index")})
    assert got["a"].dtype == torch.bfloat16 and got["b"].dtype == torch.float32
    assert got["i"].dtype == torch.int32
    with pytest.raises(ModelLoadError, match="no model.safetensors"):
        read_tensors(str(tmp_path / "void"), {})


def test_bf16_conversion_bits():
    x = torch.tensor([1.0, 0.0, -2.5, 3.1415927], dtype=torch.float32)
    bits = f32_to_bf16_bits(x)
    assert bits[0] == 0x3F80 and bits[1] == 0
    assert torch.equal(bf16_bits_to_f32(bits), x.to(torch.bfloat16).float())
    ties = torch.tensor([0x3F808000, 0x3F818000, 0x3F808001], dtype=torch.int64).to(torch.int32).view(torch.float32)
    assert f32_to_bf16_bits(ties).tolist() == [0x3F80, 0x3F82, 0x3F81]


def test_names_are_normalised_and_fused_tensors_cut(model_root, tmp_path):
    """The spellings the reference's loader accepts (bc/loader_common.rs:423-451, 475-566) and its
    fused q/k/v and gate/up tensors (:1469-1528) give the same weights as the plain names."""
    from herbert_rs_amd.models.qwen3 import NAMES
    canonical_name = NAMES.canonical
    assert canonical_name("language_model.model.layers.0.mlp.up_proj.weight") == "model.layers.0.mlp.up_proj.weight"
    assert canonical_name("language_model.lm_head.weight") == "lm_head.weight"
    assert canonical_name("model.language_model.norm.weight") == "model.norm.weight"
    assert canonical_name("layers.3.self_attn.out_proj.weight") == "model.layers.3.self_attn.o_proj.weight"
    assert canonical_name("model.layers.1.self_attn.q_proj.base_layer.weight") == "model.layers.1.self_attn.q_proj.weight"
    assert canonical_name("model.layers.1.feed_forward.w3.weight") == "model.layers.1.mlp.up_proj.weight"
    assert canonical_name("model.layers.1.ffn_norm.weight") == "model.layers.1.post_attention_layernorm.weight"

    src = make_folder(model_root, "B", "float32")
    plain = load_file(os.path.join(src, "model.safetensors"))
    other = {}
    for name, t in plain.items():
        if any(part in name for part in (".self_attn.q_proj.", ".self_attn.k_proj.", ".self_attn.v_proj.",
                                         ".mlp.gate_proj.", ".mlp.up_proj.")):
            continue
        other[name.replace("model.", "model.language_model.", 1).replace("o_proj", "out_proj")] = t
    for l in range(3):
        p = f"model.layers.{l}."
        other[f"model.language_model.layers.{l}.self_attn.qkv_proj.weight"] = torch.cat(
            [plain[p + f"self_attn.{x}_proj.weight"] for x in "qkv"], 0)
        other[f"model.language_model.layers.{l}.mlp.gate_up_proj.weight"] = torch.cat(
            [plain[p + "mlp.gate_proj.weight"], plain[p + "mlp.up_proj.weight"]], 0)
    save_file(other, str(tmp_path / "model.safetensors"))
    got = read_tensors(str(tmp_path), needs_of(TINY_B), name_map=NAMES)
    assert set(got) == set(plain) and all(torch.equal(got[k], plain[k]) for k in plain)
    # the spellings are the architecture's: the reader alone takes names as they are stored
    with pytest.raises(ModelLoadError, match="missing"):
        read_tensors(str(tmp_path), needs_of(TINY_B))
    assert resolve_architecture(TINY_B).name_map is NAMES
    # one tensor by its own name, also out of a fused one
    from herbert_rs_amd.weights import read_tensor
    for name in ("model.layers.2.self_attn.k_proj.weight", "model.layers.1.mlp.up_proj.weight", "model.norm.weight"):
        assert torch.equal(read_tensor(str(tmp_path), name, needs_of(TINY_B), NAMES), plain[name])
    with pytest.raises(ModelLoadError, match="no tensor"):
        read_tensor(str(tmp_path), "model.layers.9.mlp.up_proj.weight", needs_of(TINY_B), NAMES)
    other["model.language_model.layers.0.self_attn.qkv_proj.weight"] = torch.zeros(10, 96)
    save_file(other, str(tmp_path / "model.safetensors"))
    with pytest.raises(ModelLoadError, match=r"qkv_proj.weight: expected \[320, 96\], got \[10, 96\]"):
        read_tensors(str(tmp_path), needs_of(TINY_B), name_map=NAMES)


def test_keys_that_contradict_what_the_architecture_fixes_are_refused():
    """The reference never reads attention_bias, mlp_bias or hidden_act (biases and the activation are
    fixed for the family: crates/core/src/config.rs:508-512, loader_common.rs:853) and would run a
    model that sets them otherwise wrongly; here such a config.json is an error, and the values that
    the public Qwen3 checkpoints carry are accepted."""
    ok = dict(TINY_A, attention_bias=False, hidden_act="silu", attention_dropout=0.0, use_cache=True,
              sliding_window=None, use_sliding_window=False, max_window_layers=2, torch_dtype="bfloat16",
              rope_scaling=None, bos_token_id=1, initializer_range=0.02)
    cfg = resolve_architecture(ok).config_class.from_dict(ok)
    assert cfg.hidden_size == TINY_A["hidden_size"] and cfg.layer_windows == (None, None)
    for key, value, text in (("attention_bias", True, "no biases"), ("mlp_bias", True, "no biases"),
                             ("hidden_act", "gelu", "silu")):
        with pytest.raises(ConfigError, match=text):
            resolve_architecture(ok).config_class.from_dict(dict(ok, **{key: value}))


def counter_values(key, first, count, scale, offset):
    """The random weights' formula in NumPy, written from its description alone: the bytes of
    splitmix64(key, i) summed and centred, one float32 product, one float32 sum."""
    mask = (1 << 64) - 1
    sums = []
    for i in range(first, first + count):
        z = (key + (i + 1) * 0x9E3779B97F4A7C15) & mask
        z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & mask
        z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & mask
        z ^= z >> 31
        sums.append(sum((z >> (8 * b)) & 255 for b in range(8)) - 1020)
    scaled = np.array(sums, dtype=np.float32) * np.float32(scale)
    return (np.float32(offset) + scaled).astype(np.float32)


def test_random_weights_are_a_function_of_seed_name_and_index():
    """The host's values are the formula's, bit for bit, as float32 and rounded to bfloat16 (nearest,
    ties to even); a tensor drawn in pieces is the tensor drawn whole; the deviates are near normal;
    tensors do not depend on each other, norm weights with norm_std 0 are exactly 1."""
    from herbert_rs_amd.weights import TensorNeed, random_tensors
    from herbert_rs_amd.weights import random_init as ri
    from .plain.sampler import f32_to_bf16_bits
    key, n = 0x1234567890ABCDEF, 3000
    assert counter_values(12345, 0, 4, 1.0, 0.0).tolist() == [-196.0, 342.0, -60.0, -390.0]     # by hand, in integers
    for scale, offset in ((0.02 / ri.BYTE_SUM_SIGMA, 0.0), (0.1 / ri.BYTE_SUM_SIGMA, 1.0)):
        want = counter_values(key, 0, n, scale, offset)
        got = ri.counter_fill(torch.empty(n, dtype=torch.float32), key, scale, offset)
        assert np.array_equal(got.numpy().view(np.uint32), want.view(np.uint32))
        half = ri.counter_fill(torch.empty(n, dtype=torch.bfloat16), key, scale, offset)
        assert half.view(torch.int16).numpy().astype(np.uint16).tolist() == [f32_to_bf16_bits(v) for v in want]
        tail = ri.counter_fill(torch.empty(n - 1000, dtype=torch.float32), key, scale, offset, first=1000)
        assert torch.equal(tail, got[1000:])
    many = ri.counter_fill(torch.empty(1 << 20, dtype=torch.float32), 99, 1.0 / ri.BYTE_SUM_SIGMA).double()
    assert abs(float(many.mean())) < 0.005 and abs(float(many.std()) - 1.0) < 0.005
    assert abs(float((many ** 4).mean()) - 2.85) < 0.03 and float(many.abs().max()) <= 4.88
    assert 0.66 < float((many.abs() < 1).double().mean()) < 0.70
    needs = {"a.weight": TensorNeed((40, 24)), "n.weight": TensorNeed((24,), "scale")}
    both = random_tensors(needs, 7, "float32", std=0.05, norm_std=0.0)
    alone = random_tensors({"a.weight": needs["a.weight"]}, 7, "float32", std=0.05)
    assert torch.equal(both["a.weight"], alone["a.weight"]) and bool((both["n.weight"] == 1.0).all())
    other = random_tensors(needs, 8, "float32", std=0.05, norm_std=0.1)
    assert not torch.equal(other["a.weight"], both["a.weight"]) and 0.05 < float(other["n.weight"].std()) < 0.2
    want = counter_values(ri._tensor_seed(7, "a.weight"), 0, 960, 0.05 / ri.BYTE_SUM_SIGMA, 0.0)
    assert np.array_equal(both["a.weight"].numpy().ravel(), want)


def test_an_architecture_brings_its_own_names_default_and_initialisers(tmp_path):
    """What is particular to an architecture sits in its registry entry: the spellings of its
    checkpoints, whether it is the one taken when config.json names none, its chat format; and a
    tensor of a kind the library does not know (here a bias) brings its own random initialiser."""
    from herbert_rs_amd.config import ChatFormat, register_architecture
    from herbert_rs_amd.config import registry
    from herbert_rs_amd.weights import TensorNeed, random_tensors
    from herbert_rs_amd.weights.names import NameMap

    def small_bias(shape, gen, device, std, norm_std):
        return 0.5 + 0.01 * torch.randn(shape, generator=gen, dtype=torch.float32, device=device)

    needs = {"h.0.w": TensorNeed((4, 6)), "h.0.b": TensorNeed((4,), "bias", init=small_bias),
             "wte": TensorNeed((10, 6), "table"), "ln": TensorNeed((6,), "scale")}
    t = random_tensors(needs, 5, "bfloat16", std=0.02, norm_std=0.0)
    assert t["h.0.b"].dtype == torch.bfloat16 and abs(float(t["h.0.b"].float().mean()) - 0.5) < 0.05
    assert float(t["ln"].float().min()) == 1.0 and float(t["h.0.w"].float().abs().max()) < 0.2
    with pytest.raises(ConfigError, match="no initialiser"):
        random_tensors({"x": TensorNeed((3,), "bias")}, 0)
    with pytest.raises(ConfigError, match="made"):
        random_tensors({"x": TensorNeed((3,), "bias", init=lambda *a: torch.zeros(2))}, 0)

    names = NameMap(prefixes=(("transformer.", ""),), layer_prefix="h.",
                    layer_aliases={"weight": "w", "bias": "b"}, fused={})
    assert names.canonical("transformer.h.0.weight") == "h.0.w"
    assert names.canonical("transformer.wte") == "wte" and names.canonical("other") == "other"
    save_file({"transformer.h.0.weight": t["h.0.w"], "transformer.h.0.bias": t["h.0.b"],
               "transformer.wte": t["wte"], "ln": t["ln"], "transformer.extra": torch.zeros(1)},
              str(tmp_path / "model.safetensors"))
    ignored = []
    got = read_tensors(str(tmp_path), needs, name_map=names, ignored=ignored)
    assert all(torch.equal(got[k], t[k]) for k in needs) and ignored == ["transformer.extra"]

    saved = (dict(registry._ARCHITECTURES), dict(registry._MODEL_TYPES), list(registry._DEFAULT))
    try:
        chat = ChatFormat(lambda user, system=None: f"[{system or ''}|{user}]", "<eot>", 3)
        arch = register_architecture("ToyLM", dict, lambda cfg: None, ("toy",), name_map=names, chat=chat)
        assert resolve_architecture({"model_type": "toy"}) is arch and arch.name_map is names
        assert arch.chat.build_prompt("hi") == "[|hi]" and arch.chat.end_of_turn_id == 3
        assert resolve_architecture({}).name == "Qwen3ForCausalLM"      # registered as the default
        registry._DEFAULT[:] = []
        with pytest.raises(ConfigError, match="names neither"):
            resolve_architecture({})
    finally:
        registry._ARCHITECTURES.clear(); registry._ARCHITECTURES.update(saved[0])
        registry._MODEL_TYPES.clear(); registry._MODEL_TYPES.update(saved[1])
        registry._DEFAULT[:] = saved[2]
    qwen = resolve_architecture({"model_type": "qwen3"})
    assert qwen.chat.end_of_turn == "<|im_end|>" and qwen.chat.end_of_turn_id == 151645
    assert qwen.chat.build_prompt("Hi", "Be brief") == \
        "<|im_start|>system\nBe brief<|im_end|>\n<|im_start|>user\nHi<|im_end|>\n<|im_start|>assistant\n"


def test_plugins_named_in_the_environment_are_imported_once(tmp_path, monkeypatch):
    """HERBERT_PLUGINS names modules outside the package that register parts or architectures of
    their own; they are imported before a config.json's architecture is looked up, once, and one
    that cannot be imported is a clear error."""
    import sys
    from herbert_rs_amd.config import registry
    (tmp_path / "counting_plugin.py").write_text("import os\nos.environ['COUNTING_PLUGIN'] = str(int(os.environ.get('COUNTING_PLUGIN', '0')) + 1)\n")
    monkeypatch.syspath_prepend(str(tmp_path))
    monkeypatch.setenv("HERBERT_PLUGINS", " counting_plugin ,")
    monkeypatch.setenv("COUNTING_PLUGIN", "0")
    monkeypatch.setattr(registry, "_plugins_loaded", [])
    assert resolve_architecture({"model_type": "qwen3"}).name == "Qwen3ForCausalLM"
    assert resolve_architecture({"model_type": "qwen3"}).name == "Qwen3ForCausalLM"
    import os
    assert os.environ["COUNTING_PLUGIN"] == "1"
    monkeypatch.setenv("HERBERT_PLUGINS", "counting_plugin,no_such_plugin_module")
    with pytest.raises(ConfigError, match="no_such_plugin_module"):
        resolve_architecture({"model_type": "qwen3"})
    sys.modules.pop("counting_plugin", None)
