"""Plain whole-sequence Qwen3 forward pass and greedy generation.

It reads a model folder by itself (config.json as a dict, model.safetensors
through the safetensors package) and shares nothing with the engine.
Paths cited are relative to the reference's root; `bc/` =
crates/backends/backend_common/src/.
"""
import json
import os

import numpy as np
import torch
from safetensors import safe_open

from . import ops


def read_folder(folder, dtype=torch.float32):
    """config.json as a dict and every tensor widened to `dtype`."""
    with open(os.path.join(folder, "config.json")) as f:
        cfg = json.load(f)
    tensors = {}
    with safe_open(os.path.join(folder, "model.safetensors"), framework="pt") as f:
        for name in f.keys():
            tensors[name] = f.get_tensor(name).to(dtype)
    return cfg, tensors


def layer_window(cfg, layer):
    """Window of a layer from the public Qwen3 config keys; None = all keys.

    The reference never reads these keys (crates/core/src/config.rs:182-255
    lists what it parses), so this is parity unpinned.
    """
    types = cfg.get("layer_types")
    if types is not None:
        sliding = types[layer] == "sliding_attention"
    else:
        sliding = bool(cfg.get("use_sliding_window", False)) and \
            layer >= cfg.get("max_window_layers", cfg["num_hidden_layers"])
    if sliding and cfg.get("sliding_window"):
        return int(cfg["sliding_window"])
    return None


def rope_scaling(cfg):
    """crates/core/src/config.rs:547-580: rope_parameters, else rope_scaling; `rope_type`, else `type`;
    linear only with a factor above 1; yarn's defaults: factor 1, original = max_position_embeddings,
    beta_fast 32, beta_slow 1; anything else is the plain rotation."""
    holder = cfg.get("rope_parameters") or cfg.get("rope_scaling")
    if not isinstance(holder, dict):
        return None
    kind = holder.get("rope_type", holder.get("type"))
    factor = float(holder.get("factor", 1.0))
    if kind == "linear" and factor > 1.0:
        return {"type": "linear", "factor": factor}
    if kind == "yarn":
        return {"type": "yarn", "factor": factor,
                "original_max_position_embeddings": holder.get("original_max_position_embeddings",
                                                               cfg["max_position_embeddings"]),
                "beta_fast": float(holder.get("beta_fast", 32.0)), "beta_slow": float(holder.get("beta_slow", 1.0))}
    return None


def decoder_layer(x, positions, cfg, w, layer):
    """Pre-norm block: x + attn(norm1(x)), then x + mlp(norm2(x)).

    bc/generic_layer.rs:1149-1151 (norm1), :1234-1236 (residual 1),
    :1246-1248 (norm2), :1272-1274 (residual 2); attention steps in order
    bc/generic_attention/prefill/mod.rs:73-77 (q, k, v), :115-177 (head norms),
    :189-210 (RoPE at absolute positions), :293 (o projection).
    """
    p = f"model.layers.{layer}."
    nq = cfg["num_attention_heads"]
    nkv = cfg["num_key_value_heads"]
    hd = cfg.get("head_dim") or cfg["hidden_size"] // nq
    eps = cfg.get("rms_norm_eps", 1e-5)
    theta = cfg["rope_theta"]
    # crates/core/src/config.rs:518-525: rotary_ndims = (head_dim as f32 * partial_rotary_factor) as usize
    rot = int(np.float32(hd) * np.float32(cfg.get("partial_rotary_factor", 1.0)))

    y = ops.rms_norm(x, w[p + "input_layernorm.weight"], eps)
    q = ops.split_heads(ops.linear(y, w[p + "self_attn.q_proj.weight"]), nq, hd)
    k = ops.split_heads(ops.linear(y, w[p + "self_attn.k_proj.weight"]), nkv, hd)
    v = ops.split_heads(ops.linear(y, w[p + "self_attn.v_proj.weight"]), nkv, hd)
    q = ops.head_rms_norm(q, w[p + "self_attn.q_norm.weight"], eps)
    k = ops.head_rms_norm(k, w[p + "self_attn.k_norm.weight"], eps)
    q = ops.apply_rope(q, positions, theta, rot, rope_scaling(cfg))
    k = ops.apply_rope(k, positions, theta, rot, rope_scaling(cfg))
    a = ops.causal_attention(q, k, v, positions, window=layer_window(cfg, layer))
    a = a.reshape(a.shape[0], nq * hd)
    x = x + ops.linear(a, w[p + "self_attn.o_proj.weight"])

    y = ops.rms_norm(x, w[p + "post_attention_layernorm.weight"], eps)
    x = x + ops.swiglu_mlp(y, w[p + "mlp.gate_proj.weight"], w[p + "mlp.up_proj.weight"],
                           w[p + "mlp.down_proj.weight"])
    return x


def forward(cfg, w, tokens, start_pos=0, rows=None):
    """Logits [T, V] at every position of one whole sequence, or, with `rows`, at those positions
    only: the final norm and the head then run on those rows alone, as the reference runs them
    on the rows it needs (bc/generic_model.rs:269-274).

    Embedding without multiplier (bc/generic_model.rs:163-175), the layers in
    order (:203-219), final RMSNorm and lm_head (:266-283); the head is the
    embedding when tie_word_embeddings (default true,
    crates/core/src/config.rs:199-202; bc/loader_common.rs:1851-1872).
    """
    dtype = w["model.embed_tokens.weight"].dtype
    positions = list(range(start_pos, start_pos + len(tokens)))
    if positions and positions[-1] >= cfg["max_position_embeddings"]:
        raise ValueError("sequence exceeds max_position_embeddings")
    x = ops.embedding(tokens, w["model.embed_tokens.weight"]).to(dtype)
    for layer in range(cfg["num_hidden_layers"]):
        x = decoder_layer(x, positions, cfg, w, layer)
    if rows is not None:
        x = x[list(rows)]
    x = ops.rms_norm(x, w["model.norm.weight"], cfg.get("rms_norm_eps", 1e-5))
    head = w["model.embed_tokens.weight"] if cfg.get("tie_word_embeddings", True) \
        else w["lm_head.weight"]
    return ops.linear(x, head)


def greedy(cfg, w, prompt, max_new, stop_ids=()):
    """Greedy continuation by running the whole sequence again for each token.

    First maximal index wins (crates/core/src/sampler.rs:244-254); a stop
    token is kept in the output and ends it (crates/cli/src/main.rs:1272,
    1357-1359).
    """
    seq = list(prompt)
    out = []
    for _ in range(max_new):
        logits = forward(cfg, w, seq)[-1]
        nxt = argmax(logits)
        out.append(nxt)
        seq.append(nxt)
        if nxt in stop_ids:
            break
    return out


def argmax(logits):
    """First index of the largest value (strict >); crates/core/src/sampler.rs:244-254."""
    best, best_val = 0, float("-inf")
    for i, v in enumerate(logits.tolist()):
        if v > best_val:
            best, best_val = i, v
    return best
