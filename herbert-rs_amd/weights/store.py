"""Reading safetensors by tensor name and checking them against a model's needs.

The files are found as the reference finds them (model.safetensors.index.json
naming the shards by basename, else a single model.safetensors:
bc/loader_common.rs:1131-1149, `bc/` = crates/backends/backend_common/src/).
Tensors keep what they are stored in: bfloat16 stays bfloat16, a 32-bit float
stays so, other floats become bfloat16, integers become int32. Names are normalised and fused q/k/v and gate/up tensors are cut
into their parts as the reference's loader does (bc/loader_common.rs:423-451, 475-566, 1469-1528). Unlike the
reference, which ignores unknown names and does not check plain shapes
(bc/loader_common.rs:679-685), every problem is collected and reported in one
error: missing names, unexpected names and wrong shapes.
"""
import json
import os

import torch
from safetensors import safe_open

from ..errors import ModelLoadError

# ---- names as the reference's loader normalises them (bc/loader_common.rs:423-451, 475-566)
_ALIASES = {
    "self_attn.out_proj.weight": "self_attn.o_proj.weight",
    "self_attn.q_layernorm.weight": "self_attn.q_norm.weight",
    "self_attn.k_layernorm.weight": "self_attn.k_norm.weight",
    "operator_norm.weight": "input_layernorm.weight",
    "ffn_norm.weight": "post_attention_layernorm.weight",
    "feed_forward.w1.weight": "mlp.gate_proj.weight",
    "feed_forward.w3.weight": "mlp.up_proj.weight",
    "feed_forward.w2.weight": "mlp.down_proj.weight",
}
# fused tensors and the tensors their rows are cut into, in order (bc/loader_common.rs:1469-1528)
_FUSED = {
    "self_attn.qkv_proj.weight": ("self_attn.q_proj.weight", "self_attn.k_proj.weight",
                                  "self_attn.v_proj.weight"),
    "mlp.gate_up_proj.weight": ("mlp.gate_proj.weight", "mlp.up_proj.weight"),
}


def canonical_name(name):
    """A stored tensor's name in the form the models ask for: `model.` prefix variants of
    vision-language and bare checkpoints, the `.base_layer.weight` suffix and the aliases of
    other exporters are brought to the one spelling."""
    if name.startswith("language_model.model."):
        name = "model." + name[len("language_model.model."):]
    elif name.startswith("language_model."):
        name = name[len("language_model."):]
    elif name.startswith("model.language_model."):
        name = "model." + name[len("model.language_model."):]
    elif not name.startswith(("model.", "lm_head.")) and \
            name.startswith(("embed_tokens.", "embedding_norm.", "layers.", "norm.")):
        name = "model." + name
    if name.endswith(".base_layer.weight"):
        name = name[:-len(".base_layer.weight")] + ".weight"
    if name.startswith("model.layers."):
        head, _, rest = name[len("model.layers."):].partition(".")
        if rest in _ALIASES:
            name = f"model.layers.{head}.{_ALIASES[rest]}"
    return name


def _fused_targets(name, needs):
    """For a fused tensor's (canonical) name: the names its rows are cut into, if the model asks
    for all of them; else None."""
    for suffix, parts in _FUSED.items():
        if name.endswith("." + suffix):
            prefix = name[:-len(suffix)]
            targets = [prefix + p for p in parts]
            if all(t in needs for t in targets):
                return targets
    return None


_FLOATS = (torch.float16, torch.float64)
_INTS = (torch.int8, torch.int16, torch.int64, torch.uint8)


def shard_files(folder):
    """Paths of the safetensors files of a model folder."""
    index = os.path.join(folder, "model.safetensors.index.json")
    if os.path.exists(index):
        with open(index) as f:
            weight_map = json.load(f).get("weight_map", {})
        names = sorted({os.path.basename(v) for v in weight_map.values()})
        if not names:
            raise ModelLoadError(f"{index} names no shard")
        return [os.path.join(folder, n) for n in names]
    single = os.path.join(folder, "model.safetensors")
    if not os.path.exists(single):
        raise ModelLoadError(f"no model.safetensors (or index) in {folder}")
    return [single]


def stored_dtype(t):
    """The dtype a stored tensor is kept in."""
    if t.dtype in (torch.bfloat16, torch.float32, torch.int32):
        return t.dtype
    if t.dtype in _FLOATS:
        return torch.bfloat16
    if t.dtype in _INTS:
        return torch.int32
    raise ModelLoadError(f"unsupported dtype {t.dtype}")


def read_tensors(folder, needs, device="cpu"):
    """dict name -> tensor on `device` for exactly the names in `needs`.

    `needs` maps a name to a TensorNeed. Raises one ModelLoadError that lists
    every missing name, every unexpected name and every wrong shape.
    """
    found = {}
    unexpected = []
    wrong = []
    duplicate = []
    for path in shard_files(folder):
        try:
            handle = safe_open(path, framework="pt", device="cpu")
        except Exception as e:  # the file's own parse errors
            raise ModelLoadError(f"cannot read {path}: {e}") from None
        with handle as f:
            for stored in f.keys():
                name = canonical_name(stored)
                targets = None if name in needs else _fused_targets(name, needs)
                if name not in needs and targets is None:
                    unexpected.append(stored)
                    continue
                if any(n in found for n in (targets or [name])):
                    duplicate.append(stored)
                    continue
                shape = tuple(f.get_slice(stored).get_shape())
                if targets is None:
                    expected = tuple(needs[name].shape)
                else:       # the parts' rows one after the other
                    expected = (sum(needs[t].shape[0] for t in targets),) + tuple(needs[targets[0]].shape[1:])
                if shape != expected:
                    wrong.append(f"{stored}: expected {list(expected)}, got {list(shape)}")
                    for n in (targets or [name]):
                        found[n] = None
                    continue
                t = f.get_tensor(stored)
                try:
                    t = t.to(stored_dtype(t))
                except ModelLoadError as e:
                    wrong.append(f"{stored}: {e}")
                    for n in (targets or [name]):
                        found[n] = None
                    continue
                if targets is None:
                    found[name] = t.to(device)
                else:
                    row = 0
                    for n in targets:
                        rows = needs[n].shape[0]
                        found[n] = t[row:row + rows].contiguous().to(device)
                        row += rows
    missing = [n for n in needs if n not in found]
    if missing or unexpected or wrong or duplicate:
        parts = [f"weights in {folder} do not fit the configuration:"]
        if missing:
            parts.append(f"  missing ({len(missing)}): " + ", ".join(sorted(missing)))
        if unexpected:
            parts.append(f"  unexpected ({len(unexpected)}): " + ", ".join(sorted(unexpected)))
        if wrong:
            parts.append(f"  wrong shape or dtype ({len(wrong)}): " + "; ".join(wrong))
        if duplicate:
            parts.append(f"  stored twice ({len(duplicate)}): " + ", ".join(sorted(duplicate)))
        raise ModelLoadError("\n".join(parts))
    return found


def read_tensor(folder, name, needs):
    """The one tensor `name` of `needs` as `folder` stores it (cut out of a fused tensor if that is
    how it is stored), on the CPU."""
    if name not in needs:
        raise ModelLoadError(f"the model has no tensor {name!r}; it has: " + ", ".join(sorted(needs)))
    for path in shard_files(folder):
        with safe_open(path, framework="pt", device="cpu") as f:
            for stored in f.keys():
                cname = canonical_name(stored)
                if cname == name:
                    t = f.get_tensor(stored)
                    return t.to(stored_dtype(t))
                targets = _fused_targets(cname, needs)
                if targets and name in targets:
                    t = f.get_tensor(stored)
                    row = sum(needs[n].shape[0] for n in targets[:targets.index(name)])
                    return t[row:row + needs[name].shape[0]].contiguous().to(stored_dtype(t))
    raise ModelLoadError(f"{folder} holds no tensor {name!r}")
