"""RMSNorm as the reference computes it (crates/backends/backend_common/src/kernels.rs:54-64):
y = x / sqrt(mean(x^2) + eps) * w, the weight used as stored (not 1 + w)."""
from ..kernels import ops
from ..weights import TensorNeed
from .base import Part
from .registry import register


@register("norm", "rmsnorm")
class RMSNorm(Part):
    graph_safe = True
    hands_on = True      # y = x * w / rms(x): a product may apply the 1 / rms to its sums instead (NormedRows)

    def __init__(self, size, eps, weight):
        self.size = int(size)
        self.eps = float(eps)
        self.weight_name = weight
        self.w = None

    def tensor_needs(self):
        return {self.weight_name: TensorNeed((self.size,), "scale")}

    def load(self, tensors, rt):
        self.w = rt.weight(tensors[self.weight_name], matrix=False)

    def forward(self, ctx, x, rows=None, name="normed"):
        n = x.shape[0] if rows is None else rows.shape[0]
        y = ctx.rt.buffer(name, (n, self.size))
        ops.rmsnorm(x, self.w, y, self.eps, rows)
        return y
