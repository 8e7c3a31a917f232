"""The tiny configurations the tests run and helpers to make their model folders.

A and B are the two configurations the benchmark description names; C adds what
they lack: one kv head, a head size that is no power of two, and a window on one
of its layers (long enough sequences cross its edge and give pages back).
They differ in every size and option. D has the head size of the large models (128), for which
the bfloat16 engine has kernels of its own (long prompts, decoding) that the others never reach.
"""
import os

import torch

from herbert_rs_amd.config.registry import resolve_architecture
from herbert_rs_amd.engine.model import Model
from herbert_rs_amd.weights import write_model_folder

TINY_A = dict(
    architectures=["Qwen3ForCausalLM"], model_type="qwen3",
    num_hidden_layers=2, hidden_size=64, num_attention_heads=4, num_key_value_heads=2, head_dim=16,
    intermediate_size=128, vocab_size=256, rope_theta=10000.0, rms_norm_eps=1e-6,
    tie_word_embeddings=True, max_position_embeddings=128, eos_token_id=255)
TINY_B = dict(
    architectures=["Qwen3ForCausalLM"], model_type="qwen3",
    num_hidden_layers=3, hidden_size=96, num_attention_heads=6, num_key_value_heads=2, head_dim=32,
    intermediate_size=224, vocab_size=384, rope_theta=1000000.0, rms_norm_eps=1e-5,
    tie_word_embeddings=False, max_position_embeddings=256, eos_token_id=[383, 7])
TINY_C = dict(
    architectures=["Qwen3ForCausalLM"], model_type="qwen3",
    num_hidden_layers=2, hidden_size=80, num_attention_heads=5, num_key_value_heads=1, head_dim=48,
    intermediate_size=176, vocab_size=320, rope_theta=500000.0, rms_norm_eps=3e-6,
    tie_word_embeddings=False, max_position_embeddings=512, eos_token_id=3,
    sliding_window=70, layer_types=["sliding_attention", "full_attention"])

TINY_D = dict(
    architectures=["Qwen3ForCausalLM"], model_type="qwen3",
    num_hidden_layers=2, hidden_size=192, num_attention_heads=4, num_key_value_heads=2, head_dim=128,
    intermediate_size=320, vocab_size=512, rope_theta=1000000.0, rms_norm_eps=1e-6,
    tie_word_embeddings=True, max_position_embeddings=2048, eos_token_id=511)

# eight kv heads of 64: a step of a few thousand prompt tokens has enough attention tiles for the
# kernel that long prompts take
TINY_F = dict(
    architectures=["Qwen3ForCausalLM"], model_type="qwen3",
    num_hidden_layers=1, hidden_size=128, num_attention_heads=8, num_key_value_heads=8, head_dim=64,
    intermediate_size=160, vocab_size=288, rope_theta=1000000.0, rms_norm_eps=1e-6,
    tie_word_embeddings=True, max_position_embeddings=4096, eos_token_id=1)

CONFIGS = {"A": (TINY_A, 0, 0.02), "B": (TINY_B, 1, 0.05), "C": (TINY_C, 2, 0.04), "D": (TINY_D, 3, 0.05), "F": (TINY_F, 5, 0.05)}


def spec_of(raw):
    arch = resolve_architecture(raw)
    cfg = arch.config_class.from_dict(raw)
    return cfg, arch.build_spec(cfg)


def make_folder(root, name, dtype="float32", overrides=None, seed=None, std=None):
    """Write the random model `name` (A, B or C) into root/<name>_<dtype> once; returns the path."""
    raw, seed0, std0 = CONFIGS[name]
    raw = dict(raw)
    tag = f"{name}_{dtype}"
    if overrides:
        raw.update(overrides)
        tag += "_" + "".join(c if c.isalnum() or c in "._-" else "-" for c in
                             "_".join(f"{k}{v}" for k, v in sorted(overrides.items())))
    folder = os.path.join(str(root), tag)
    if os.path.exists(os.path.join(folder, "model.safetensors")):
        return folder
    cfg, spec = spec_of(raw)
    needs = Model(spec).tensor_needs()
    write_model_folder(folder, raw, needs, seed if seed is not None else seed0, dtype=dtype,
                       std=std if std is not None else std0, norm_std=0.1)
    return folder


def random_tokens(vocab, n, seed):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, vocab, (n,), generator=g).tolist()


def make_folder_from(root, tag, raw, seed, dtype="float32", std=0.02, norm_std=0.1):
    """Write a random model of the configuration `raw` into root/<tag>_<dtype> once; returns the path."""
    folder = os.path.join(str(root), f"{tag}_{dtype}")
    if os.path.exists(os.path.join(folder, "model.safetensors")):
        return folder
    cfg, spec = spec_of(raw)
    write_model_folder(folder, dict(raw), Model(spec).tensor_needs(), seed, dtype=dtype, std=std,
                       norm_std=norm_std)
    return folder
