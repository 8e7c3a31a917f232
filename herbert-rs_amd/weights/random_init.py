"""Seeded random weights: as tensors, or written out as a model folder.

The reference has no such mode. Matrices and the embedding table are
N(0, std); norm weights are 1 + N(0, norm_std). Each tensor has a generator
of its own, seeded from the seed and the tensor's name, so a tensor's values
do not depend on which other tensors exist.
"""
import hashlib
import json
import os

import torch
from safetensors.torch import save_file

from ..errors import ConfigError

_DTYPES = {"float32": torch.float32, "bfloat16": torch.bfloat16,
           torch.float32: torch.float32, torch.bfloat16: torch.bfloat16}


def _tensor_seed(seed, name):
    digest = hashlib.sha256(f"{seed}:{name}".encode()).digest()
    return int.from_bytes(digest[:8], "little") & ((1 << 63) - 1)


def _draw_index(shape, gen, device, std, norm_std):
    return torch.zeros(shape, dtype=torch.int32, device=device)


def _draw_scale(shape, gen, device, std, norm_std):
    t = torch.ones(shape, dtype=torch.float32, device=device)
    if norm_std:
        t += norm_std * torch.randn(shape, generator=gen, dtype=torch.float32, device=device)
    return t


# how a role is drawn when the need brings no initialiser of its own; "matrix" and "table" are
# drawn below (in row blocks when large)
ROLE_INITIALISERS = {"index": _draw_index, "scale": _draw_scale}


def random_tensor(name, need, seed, dtype, std=0.02, norm_std=0.0, device="cpu"):
    """One tensor for `need`, drawn in float32 on `device` and stored as `dtype` (integers stay
    int32). The need's own initialiser decides if it has one, else its role."""
    gen = torch.Generator(device=device)
    gen.manual_seed(_tensor_seed(seed, name))
    init = need.init or ROLE_INITIALISERS.get(need.role)
    if init is not None:
        t = init(tuple(need.shape), gen, device, std, norm_std)
        if tuple(t.shape) != tuple(need.shape):
            raise ConfigError(f"the initialiser of {name} made {list(t.shape)}, not {list(need.shape)}")
        return t if not t.is_floating_point() else t.to(dtype)
    if need.role not in ("matrix", "table"):
        raise ConfigError(f"tensor {name}: role {need.role!r} has no initialiser; give the TensorNeed one")
    rows = need.shape[0]
    if device == "cpu" or rows * (need.shape[1] if len(need.shape) > 1 else 1) < (1 << 28):
        t = torch.randn(need.shape, generator=gen, dtype=torch.float32, device=device)
        return t.mul_(std).to(dtype)
    # large tensors on the GPU: draw in row blocks so the float32 copy stays small
    out = torch.empty(need.shape, dtype=dtype, device=device)
    step = max(1, (1 << 27) // max(1, need.shape[1]))
    for r0 in range(0, rows, step):
        r1 = min(rows, r0 + step)
        blk = torch.randn((r1 - r0,) + tuple(need.shape[1:]), generator=gen,
                          dtype=torch.float32, device=device)
        out[r0:r1] = blk.mul_(std).to(dtype)
    return out


def random_tensors(needs, seed, dtype="bfloat16", std=0.02, norm_std=0.0, device="cpu"):
    """dict name -> tensor for every need."""
    if dtype not in _DTYPES:
        raise ConfigError(f"random weights: dtype must be float32 or bfloat16, got {dtype!r}")
    dt = _DTYPES[dtype]
    return {name: random_tensor(name, need, seed, dt, std, norm_std, device)
            for name, need in needs.items()}


def write_model_folder(folder, config_dict, needs, seed, dtype="float32", std=0.02, norm_std=0.1):
    """Write config.json and model.safetensors of a random model into `folder`."""
    os.makedirs(folder, exist_ok=True)
    tensors = random_tensors(needs, seed, dtype, std, norm_std, device="cpu")
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(config_dict, f, indent=1)
    save_file({k: v.contiguous() for k, v in tensors.items()},
              os.path.join(folder, "model.safetensors"))
    return folder
