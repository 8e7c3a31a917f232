"""Seeded random weights: as tensors, or written out as a model folder.

The reference has no such mode. Matrices and the embedding table are near N(0, std), norm weights
1 + N(0, norm_std) (the sum of eight random bytes stands for the normal deviate: bounded at 4.88
deviations, excess kurtosis -0.15). Every element is a function of the seed, the tensor's name and
the element's index alone (csrc/random_weights.hip: a splitmix64 counter), computed by a kernel
on the GPU and by the same function on the host: a model drawn on the GPU (`Engine.from_config`) and
a model folder written from the same seed (`write_model_folder`) hold the same bits, and a tensor's
values do not depend on which other tensors exist. A tensor whose need brings an initialiser of
its own is drawn by that, from a torch generator seeded the same way (such values are the
initialiser's business, and differ between CPU and GPU as torch's generators do).
"""
import ctypes
import hashlib
import json
import math
import os

import numpy as np
import torch
from safetensors.torch import save_file

from ..errors import ConfigError
from ..kernels import lib

_DTYPES = {"float32": torch.float32, "bfloat16": torch.bfloat16,
           torch.float32: torch.float32, torch.bfloat16: torch.bfloat16}
_CODES = {torch.float32: 0, torch.bfloat16: 1}

# standard deviation of the sum of eight independent bytes
BYTE_SUM_SIGMA = math.sqrt(8 * (256 ** 2 - 1) / 12)

_U64 = ctypes.c_uint64
lib.register_signatures("random_weights", {
    "hb_random_fill": [ctypes.c_void_p, ctypes.c_int, ctypes.c_size_t, _U64, _U64, ctypes.c_float, ctypes.c_float,
                       ctypes.c_void_p],
    "hb_random_fill_host": [ctypes.c_void_p, ctypes.c_int, ctypes.c_size_t, _U64, _U64, ctypes.c_float,
                            ctypes.c_float, ctypes.c_int],
})


def _tensor_seed(seed, name):
    digest = hashlib.sha256(f"{seed}:{name}".encode()).digest()
    return int.from_bytes(digest[:8], "little") & ((1 << 63) - 1)


def counter_fill(t, key, scale, offset=0.0, first=0):
    """t[i] = offset + scale * (the centred byte sum of splitmix64(key, first + i)), for a contiguous
    float32 or bfloat16 tensor on the GPU or in host memory; `scale` is used as a float32."""
    if t.dtype not in _CODES or not t.is_contiguous():
        raise ConfigError("random weights are drawn into contiguous float32 or bfloat16 tensors")
    scale = float(np.float32(scale))
    offset = float(np.float32(offset))
    if t.is_cuda:
        with torch.cuda.device(t.device):
            lib.call("random_weights", "hb_random_fill", t.data_ptr(), _CODES[t.dtype], t.numel(), int(key), int(first),
                     scale, offset, torch.cuda.current_stream().cuda_stream)
    else:
        lib.call("random_weights", "hb_random_fill_host", t.data_ptr(), _CODES[t.dtype], t.numel(), int(key),
                 int(first), scale, offset, min(16, os.cpu_count() or 1))
    return t


def _draw_index(shape, gen, device, std, norm_std):
    return torch.zeros(shape, dtype=torch.int32, device=device)


# how a role is drawn when the need brings no initialiser of its own; "matrix", "table" and "scale"
# come from the counter (below)
ROLE_INITIALISERS = {"index": _draw_index}
COUNTER_ROLES = {"matrix": lambda std, norm_std: (std, 0.0), "table": lambda std, norm_std: (std, 0.0),
                 "scale": lambda std, norm_std: (norm_std, 1.0)}


def random_tensor(name, need, seed, dtype, std=0.02, norm_std=0.0, device="cpu"):
    """One tensor for `need`: matrices and tables in `dtype`, scales (norm weights) in float32 then
    `dtype`, integers int32. The need's own initialiser decides if it has one, else its role."""
    init = need.init or ROLE_INITIALISERS.get(need.role)
    if init is not None:
        gen = torch.Generator(device=device)
        gen.manual_seed(_tensor_seed(seed, name))
        t = init(tuple(need.shape), gen, device, std, norm_std)
        if tuple(t.shape) != tuple(need.shape):
            raise ConfigError(f"the initialiser of {name} made {list(t.shape)}, not {list(need.shape)}")
        return t if not t.is_floating_point() else t.to(dtype)
    if need.role not in COUNTER_ROLES:
        raise ConfigError(f"tensor {name}: role {need.role!r} has no initialiser; give the TensorNeed one")
    deviation, offset = COUNTER_ROLES[need.role](std, norm_std)
    out = torch.empty(tuple(need.shape), dtype=dtype, device=device)
    return counter_fill(out, _tensor_seed(seed, name), deviation / BYTE_SUM_SIGMA, offset)


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
