"""How a layer's parts are arranged.

"prenorm": x += mixer(norm_input(x)); x += feed_forward(norm_post_mixer(x)), the
arrangement of the reference's two-norm layer
(crates/backends/backend_common/src/generic_layer.rs:1149-1151, 1234-1236,
1246-1248, 1272-1274).
"""
from .base import Part
from .registry import register


@register("block", "prenorm")
class PreNormBlock(Part):
    graph_safe = True

    norm_roles = ("input", "post_mixer")

    def __init__(self, mixer, feed_forward, norms):
        self.mixer = mixer
        self.feed_forward = feed_forward
        self.norms = norms
        missing = [r for r in self.norm_roles if r not in norms]
        if missing:
            raise ValueError(f"prenorm block needs norms {missing}")

    def parts(self):
        return [self.norms["input"], self.mixer, self.norms["post_mixer"], self.feed_forward]

    def first_norm(self):
        """The norm that the residual stream meets first in this block."""
        return self.norms["input"]

    def forward(self, ctx, x):
        after = ctx.norm_after_block
        self._run(ctx, x, self.norms["input"], self.mixer, (self.norms["post_mixer"], ctx.entry))
        self._run(ctx, x, self.norms["post_mixer"], self.feed_forward, after)

    @staticmethod
    def _run(ctx, x, norm, part, ahead):
        """part(norm(x)) added to x. A part may offer forward_from_residual(ctx, x, norm), which
        returns True if it has done the norm itself inside its first kernel, or has used what the
        part before left of it (ctx.handed). `ahead` is (the norm that x meets next, its entry)."""
        left, ctx.left = ctx.left, None
        valid = (left is not None and left.norm is norm and left.entry == ctx.entry
                 and left.x.data_ptr() == x.data_ptr() and left.x.shape == x.shape)
        ctx.norm_ahead = ahead
        if valid and left.squares is None:          # the product before has normed the rows as well
            ctx.handed = None
            part.forward(ctx, left.xg, x)
            return
        ctx.handed = left if valid else None
        fused = getattr(part, "forward_from_residual", None)
        if fused is not None and fused(ctx, x, norm):
            return
        ctx.handed = None
        part.forward(ctx, norm.forward(ctx, x), x)
