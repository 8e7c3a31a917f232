"""The Python entry point: load a model folder, generate from it, write a random model.

The reference has no Python; the option names and meanings are those of its command line
(crates/cli/src/main.rs:54-195).
"""
import os

from .config import load_config, read_config_json
from .config.registry import resolve_architecture
from .engine import Engine
from .engine.model import Model
from .sampling import SamplingParams
from .weights import write_model_folder


def load(model, dtype="bfloat16", cache_tokens=4096, max_slots=None):
    """The engine of a model folder (config.json + model.safetensors) on the GPU."""
    return Engine.from_folder(model, dtype=dtype, max_tokens=cache_tokens, max_slots=max_slots)


def generate(model, prompts, temperature=0.4, top_k=40, top_p=0.9, max_tokens=2048, stop_ids=(),
             ignore_eos=False, no_repeat_check=False, seed=None, dtype="bfloat16", max_batch=64,
             prefill_chunk=None, think_budget=0, think_tokens=None):
    """Generate from token-id prompts. `model` is a folder or an Engine; `prompts` one list of
    ids or a list of them. Returns the generated ids (one list, or a list of lists).
    `prefill_chunk`: prompts go through the engine in pieces of that many tokens. `think_budget`
    with `think_tokens` (sampling.ThinkTokens): a cap on the tokens of a think block."""
    single = bool(prompts) and isinstance(prompts[0], int)
    plist = [list(prompts)] if single else [list(p) for p in prompts]
    params = SamplingParams(temperature=temperature, top_k=top_k, top_p=top_p, max_tokens=max_tokens,
                            stop_ids=tuple(stop_ids), ignore_eos=ignore_eos,
                            repeat_check=not no_repeat_check, seed=seed, think_budget=think_budget,
                            think_tokens=think_tokens)
    if isinstance(model, Engine):
        engine = model
    else:
        room = sum((len(p) + max_tokens + 127) // 64 * 64 for p in plist[:max_batch])
        engine = load(model, dtype=dtype, cache_tokens=room)
    results = engine.generate(plist, params, max_batch=max_batch, prefill_chunk=prefill_chunk)
    tokens = [r.tokens for r in results]
    return tokens[0] if single else tokens


def write_random_model(folder, config, seed=0, dtype="bfloat16", std=0.02, norm_std=0.0):
    """Write config.json and model.safetensors with seeded random weights.
    `config` is a dict of config.json keys, a typed configuration or a path to a config.json."""
    if isinstance(config, (str, os.PathLike)):
        raw = read_config_json(config)
    elif isinstance(config, dict):
        raw = dict(config)
    else:
        raw = config.to_dict()
    arch = resolve_architecture(raw)
    cfg = arch.config_class.from_dict(raw)
    needs = Model(arch.build_spec(cfg)).tensor_needs()
    return write_model_folder(folder, raw, needs, seed, dtype=dtype, std=std, norm_std=norm_std)
