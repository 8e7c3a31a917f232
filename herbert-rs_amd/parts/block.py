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

    def forward(self, ctx, x):
        y = self.norms["input"].forward(ctx, x)
        self.mixer.forward(ctx, y, x)
        y = self.norms["post_mixer"].forward(ctx, x)
        self.feed_forward.forward(ctx, y, x)
