"""Dense gated feed-forward: down(silu(gate(y)) * up(y)), no biases.

crates/backends/backend_common/src/generic_mlp.rs:83-96 and kernels.rs:676-687
of the reference; gate and up are one fused matrix here so that the activations
are read once.
"""
import torch

from ..kernels import mfma, ops
from ..weights import TensorNeed
from .base import Part
from .linear import Linear
from .registry import register


@register("feed_forward", "swiglu")
class SwiGLU(Part):
    graph_safe = True

    def __init__(self, hidden_size, intermediate_size, names, shared=None):
        """names: dict with gate, up, down -> tensor names."""
        self.hidden_size = int(hidden_size)
        self.intermediate_size = int(intermediate_size)
        self.names = dict(names)
        self.gate_up = self.down = None
        self.fused_epilogue = False

    def tensor_needs(self):
        n = self.names
        return {n["gate"]: TensorNeed((self.intermediate_size, self.hidden_size)),
                n["up"]: TensorNeed((self.intermediate_size, self.hidden_size)),
                n["down"]: TensorNeed((self.hidden_size, self.intermediate_size))}

    def load(self, tensors, rt):
        n = self.names
        gate, up = rt.weight(tensors[n["gate"]]), rt.weight(tensors[n["up"]])
        # bfloat16 with sizes the MFMA kernel takes: gate and up rows interleaved so that the
        # product's epilogue applies silu(gate) * up and the float32 [T, 2I] never exists
        self.fused_epilogue = (rt.dtype == torch.bfloat16 and self.intermediate_size % 16 == 0
                               and self.hidden_size % 32 == 0 and mfma.gemm_supported(
                                   gate[:1], gate, swiglu=True))
        if self.fused_epilogue:
            self.gate_up = Linear(mfma.interleave_gate_up(gate, up), scratch=rt.scratch)
        else:
            self.gate_up = Linear(torch.cat([gate, up], 0), scratch=rt.scratch)
        self.down = Linear(rt.weight(tensors[n["down"]]), scratch=rt.scratch)

    def forward_from_residual(self, ctx, x, norm):
        """With few rows and the fused epilogue no norm kernel runs: the gate/up kernel takes what the
        product before left of the norm, or else does the norm itself on the way."""
        if not self.fused_epilogue:
            return False
        handed = ctx.take_handed(self.gate_up, x)
        if handed is not None:
            self.forward(ctx, handed.xg, x, row_scale=handed.row_scale())
            return True
        if not (hasattr(norm, "w") and hasattr(norm, "eps") and self.gate_up.fuses_norm(x)):
            return False
        self.forward(ctx, None, x, fused_norm=norm)
        return True

    def forward(self, ctx, y, x, fused_norm=None, row_scale=None):
        rt = ctx.rt
        T = x.shape[0]
        act = rt.buffer("act", (T, self.intermediate_size))
        if fused_norm is not None:
            self.gate_up.forward_swiglu(x, act, norm=(fused_norm.w, fused_norm.eps))
        elif self.fused_epilogue:
            self.gate_up.forward_swiglu(y, act, row_scale=row_scale)
        else:
            gu = rt.buffer("gate_up", (T, 2 * self.intermediate_size), torch.float32)
            self.gate_up.forward(y, gu)
            ops.swiglu(gu, act)
        left = ctx.leave_norm(self.down, x)
        self.down.forward(act, x, accumulate=True, leave=None if left is None else left.leave())
