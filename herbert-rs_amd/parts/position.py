"""Position encodings. A mixer takes one as a parameter; "none" is a valid choice.

"rope": half-split rotation with a table built as the reference builds it
(crates/backends/backend_common/src/loader_common.rs:179-202):
inv_freq_i = 1 / theta^(2i / R), angle = float32(pos) * inv_freq_i in float32,
cos and sin of it for every position below max_positions.
Scaled frequencies, all in float32 as there: "linear" divides every inv_freq by the factor
(:205-228); "yarn" keeps those whose wavelength 2 pi / inv_freq is below original_max / beta_fast,
divides by the factor those above original_max / beta_slow, and blends in between with
smooth = (original_max / wavelength - beta_slow) / (beta_fast - beta_slow) (:239-287).
"""
import math

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

    def __init__(self, theta, rotary_dims, max_positions, scaling=None):
        if rotary_dims % 2:
            raise ValueError("rotary_dims must be even")
        self.theta = float(theta)
        self.rotary_dims = int(rotary_dims)
        self.max_positions = int(max_positions)
        # (type, factor, original_max_position_embeddings, beta_fast, beta_slow)
        self.scaling = tuple(scaling) if scaling else ("default", 1.0, None, 32.0, 1.0)
        if self.scaling[0] not in ("default", "linear", "yarn"):
            raise ValueError(f"unknown rope scaling {self.scaling[0]!r}")
        self.cos = self.sin = None

    def inv_freq(self):
        half = self.rotary_dims // 2
        theta = torch.tensor(self.theta, dtype=torch.float32)
        exponent = (2.0 * torch.arange(half, dtype=torch.float32)) / float(self.rotary_dims)
        inv_freq = 1.0 / torch.pow(theta, exponent)
        kind, factor, original, beta_fast, beta_slow = self.scaling
        f32 = lambda v: torch.tensor(v, dtype=torch.float32)
        if kind == "linear":
            inv_freq = 1.0 / (torch.pow(theta, exponent) * f32(factor))
        elif kind == "yarn":
            original = f32(float(original if original is not None else self.max_positions))
            low, high = original / f32(beta_fast), original / f32(beta_slow)
            wavelen = f32(2.0) * f32(math.pi) / inv_freq
            smooth = (original / wavelen - f32(beta_slow)) / (f32(beta_fast) - f32(beta_slow))
            scaled = inv_freq / f32(factor)
            blend = (1.0 - smooth) * scaled + smooth * inv_freq
            inv_freq = torch.where(wavelen < low, inv_freq, torch.where(wavelen > high, scaled, blend))
        return inv_freq

    def load(self, tensors, rt):
        inv_freq = self.inv_freq()
        pos = torch.arange(self.max_positions, dtype=torch.float32)
        ang = pos[:, None] * inv_freq[None, :]
        self.cos = torch.cos(ang).contiguous().to(rt.device)
        self.sin = torch.sin(ang).contiguous().to(rt.device)

    def rotation(self):
        return self.cos, self.sin, self.rotary_dims
