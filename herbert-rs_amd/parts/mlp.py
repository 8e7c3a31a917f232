"""Dense gated feed-forward: down(silu(gate(y)) * up(y)), no biases.

crates/backends/backend_common/src/generic_mlp.rs:83-96 and kernels.rs:676-687
of the reference; gate and up are one fused matrix here so that the activations
are read once.
"""
import torch

from ..kernels import ops
from ..weights import TensorNeed
from .base import Part
from .linear import Linear
from .registry import register


@register("feed_forward", "swiglu")
class SwiGLU(Part):
    def __init__(self, hidden_size, intermediate_size, names, shared=None):
        """names: dict with gate, up, down -> tensor names."""
        self.hidden_size = int(hidden_size)
        self.intermediate_size = int(intermediate_size)
        self.names = dict(names)
        self.gate_up = self.down = None

    def tensor_needs(self):
        n = self.names
        return {n["gate"]: TensorNeed((self.intermediate_size, self.hidden_size)),
                n["up"]: TensorNeed((self.intermediate_size, self.hidden_size)),
                n["down"]: TensorNeed((self.hidden_size, self.intermediate_size))}

    def load(self, tensors, rt):
        n = self.names
        fused = torch.cat([tensors[n["gate"]].to(rt.device), tensors[n["up"]].to(rt.device)], 0)
        self.gate_up = Linear(rt.weight(fused))
        self.down = Linear(rt.weight(tensors[n["down"]]))

    def forward(self, ctx, y, x):
        rt = ctx.rt
        T = y.shape[0]
        gu = rt.buffer("gate_up", (T, 2 * self.intermediate_size), torch.float32)
        self.gate_up.forward(y, gu)
        act = rt.buffer("act", (T, self.intermediate_size))
        ops.swiglu(gu, act)
        self.down.forward(act, x, accumulate=True)
