"""Position encodings. A mixer takes one as a parameter; "none" is a valid choice.

"rope": half-split rotation with a table built as the reference builds it
(crates/backends/backend_common/src/loader_common.rs:179-202):
inv_freq_i = 1 / theta^(2i / R), angle = float32(pos) * inv_freq_i in float32,
cos and sin of it for every position below max_positions.
"""
import torch

from .base import Part
from .registry import register


@register("position", "none")
class NoPosition(Part):
    graph_safe = True

    def __init__(self, **_):
        pass

    def rotation(self):
        return None


@register("position", "rope")
class RotaryHalfSplit(Part):
    graph_safe = True

    def __init__(self, theta, rotary_dims, max_positions):
        if rotary_dims % 2:
            raise ValueError("rotary_dims must be even")
        self.theta = float(theta)
        self.rotary_dims = int(rotary_dims)
        self.max_positions = int(max_positions)
        self.cos = self.sin = None

    def load(self, tensors, rt):
        half = self.rotary_dims // 2
        theta = torch.tensor(self.theta, dtype=torch.float32)
        exponent = (2.0 * torch.arange(half, dtype=torch.float32)) / float(self.rotary_dims)
        inv_freq = 1.0 / torch.pow(theta, exponent)
        pos = torch.arange(self.max_positions, dtype=torch.float32)
        ang = pos[:, None] * inv_freq[None, :]
        self.cos = torch.cos(ang).contiguous().to(rt.device)
        self.sin = torch.sin(ang).contiguous().to(rt.device)

    def rotation(self):
        return self.cos, self.sin, self.rotary_dims
