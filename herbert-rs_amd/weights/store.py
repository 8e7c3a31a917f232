"""Reading safetensors by tensor name and checking them against a model's needs.

The files are found as the reference finds them (model.safetensors.index.json
naming the shards by basename, else a single model.safetensors:
bc/loader_common.rs:1131-1149, `bc/` = crates/backends/backend_common/src/).
Tensors keep what they are stored in: bfloat16 stays bfloat16, a 32-bit float
stays so, other floats become bfloat16, integers become int32. How stored
names are spelled and which tensors are fused is the architecture's NameMap
(weights/names.py); the reader applies it and knows no spelling itself.
Stored tensors that the model does not ask for are passed over, as the
reference passes them over (bc/loader_common.rs:679-685,1588: rotary
inv_freq buffers, a stored head beside tied embeddings, :1851-1872); with
`strict=True` they are an error too. Unlike the reference, which does not
check plain shapes, every other problem is collected and reported in one
error: missing names, wrong shapes or dtypes, names stored twice.
"""
import json
import os

import torch
from safetensors import safe_open

from ..errors import ModelLoadError
from .names import AS_STORED

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


def read_tensors(folder, needs, device="cpu", name_map=None, strict=False, ignored=None):
    """dict name -> tensor on `device` for exactly the names in `needs`.

    `needs` maps a name to a TensorNeed; `name_map` is the architecture's NameMap (default: names
    as stored). Raises one ModelLoadError that lists every missing name, every wrong shape and
    every name stored twice. Stored tensors nobody asks for are skipped and their names appended
    to `ignored` (a list, if given); with `strict` they are listed in the error as unexpected.
    """
    name_map = name_map or AS_STORED
    found = {}
    unexpected = ignored if ignored is not None else []
    del unexpected[:]
    wrong = []
    duplicate = []
    for path in shard_files(folder):
        try:
            handle = safe_open(path, framework="pt", device="cpu")
        except Exception as e:  # the file's own parse errors
            raise ModelLoadError(f"cannot read {path}: {e}") from None
        with handle as f:
            for stored in f.keys():
                name = name_map.canonical(stored)
                targets = None if name in needs else name_map.fused_targets(name, needs)
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
    if not strict:
        unexpected = []
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


def read_tensor(folder, name, needs, name_map=None):
    """The one tensor `name` of `needs` as `folder` stores it (cut out of a fused tensor if that is
    how it is stored), on the CPU."""
    name_map = name_map or AS_STORED
    if name not in needs:
        raise ModelLoadError(f"the model has no tensor {name!r}; it has: " + ", ".join(sorted(needs)))
    for path in shard_files(folder):
        with safe_open(path, framework="pt", device="cpu") as f:
            for stored in f.keys():
                cname = name_map.canonical(stored)
                if cname == name:
                    t = f.get_tensor(stored)
                    return t.to(stored_dtype(t))
                targets = name_map.fused_targets(cname, needs)
                if targets and name in targets:
                    t = f.get_tensor(stored)
                    row = sum(needs[n].shape[0] for n in targets[:targets.index(name)])
                    return t[row:row + needs[name].shape[0]].contiguous().to(stored_dtype(t))
    raise ModelLoadError(f"{folder} holds no tensor {name!r}")
