"""Reading safetensors by tensor name and checking them against a model's needs.

The files are found as the reference finds them (model.safetensors.index.json
naming the shards by basename, else a single model.safetensors:
bc/loader_common.rs:1131-1149, `bc/` = crates/backends/backend_common/src/).
Tensors keep what they are stored in: bfloat16 stays bfloat16, a 32-bit float
stays so, other floats become bfloat16, integers become int32. Unlike the
reference, which ignores unknown names and does not check plain shapes
(bc/loader_common.rs:679-685), every problem is collected and reported in one
error: missing names, unexpected names and wrong shapes.
"""
import json
import os

import torch
from safetensors import safe_open

from ..errors import ModelLoadError

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
            for name in f.keys():
                if name not in needs:
                    unexpected.append(name)
                    continue
                if name in found:
                    duplicate.append(name)
                    continue
                shape = tuple(f.get_slice(name).get_shape())
                if shape != tuple(needs[name].shape):
                    wrong.append(f"{name}: expected {list(needs[name].shape)}, got {list(shape)}")
                    found[name] = None
                    continue
                t = f.get_tensor(name)
                try:
                    t = t.to(stored_dtype(t))
                except ModelLoadError as e:
                    wrong.append(f"{name}: {e}")
                    found[name] = None
                    continue
                found[name] = t.to(device)
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
