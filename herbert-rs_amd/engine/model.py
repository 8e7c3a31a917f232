"""A model built from a ModelSpec: parts, their weights, and the forward pass of one step.

The forward pass follows the reference's drivers
(crates/backends/backend_common/src/generic_model.rs:131-319 for a prompt,
:524-726 for one token) but is one function for both: embed the step's tokens,
run the schedule's entries in order on the packed rows, then the final norm
and the head on the wanted rows only.
"""
from ..errors import ConfigError
from ..kernels import ops
from ..parts import StepContext, build
from ..parts.spec import ScheduleEntry


class SharedParts:
    """Parts that several layers share, built once for each distinct specification."""

    def __init__(self):
        self._positions = {}

    def position(self, spec):
        key = (spec.kind, tuple(sorted(spec.params.items())))
        if key not in self._positions:
            self._positions[key] = build("position", spec)
        return self._positions[key]

    def all(self):
        return list(self._positions.values())


class Model:
    def __init__(self, spec):
        self.spec = spec
        self.shared = SharedParts()
        self.embedding = build("embedding", spec.embedding, shared=self.shared)
        self.blocks = []
        for layer in spec.layers:
            mixer = build("mixer", layer.mixer, shared=self.shared)
            ffn = build("feed_forward", layer.feed_forward, shared=self.shared)
            norms = {role: build("norm", ns) for role, ns in layer.norms.items()}
            self.blocks.append(build("block", layer.block, mixer=mixer, feed_forward=ffn, norms=norms))
        final_norm = build("norm", spec.final_norm)
        self.head = build("head", spec.head, norm=final_norm, shared=self.shared)
        self.schedule = [e if isinstance(e, ScheduleEntry) else ScheduleEntry(*e) for e in spec.schedule]
        for i, e in enumerate(self.schedule):
            if not 0 <= e.layer < len(self.blocks):
                raise ConfigError(f"schedule entry {i} names layer {e.layer}, which does not exist")
            if e.cache is not None:
                if not 0 <= e.cache < i or self.schedule[e.cache].cache is not None:
                    raise ConfigError(f"schedule entry {i} must read the cache of an earlier entry "
                                      "that owns one")
        self.loaded = False

    # ---- weights
    def tensor_needs(self):
        needs = {}
        for part in self._weight_parts():
            for name, need in part.tensor_needs().items():
                if name in needs and needs[name] != need:
                    raise ConfigError(f"tensor {name} is asked for with two different shapes")
                needs[name] = need
        return needs

    def _weight_parts(self):
        parts = [self.embedding, self.head]
        for b in self.blocks:
            parts.extend(b.parts())
        return parts

    def load(self, tensors, rt):
        self.embedding.load(tensors, rt, shared_with_head=getattr(self.head, "tied", False))
        for p in self.shared.all():
            p.load(tensors, rt)
        for b in self.blocks:
            for p in b.parts():
                p.load(tensors, rt)
        self.head.load(tensors, rt, embedding=self.embedding)
        self.loaded = True

    @property
    def graph_safe(self):
        """True if every part only enqueues GPU work, so that a step can be captured and replayed."""
        parts = self._weight_parts() + self.blocks + self.shared.all()
        return all(getattr(p, "graph_safe", False) for p in parts)

    # ---- cache
    def cache_needs(self):
        """{schedule entry: need} for the entries that own a cache."""
        needs = {}
        for i, e in enumerate(self.schedule):
            if e.cache is None:
                need = self.blocks[e.layer].mixer.cache_need()
                if need is not None:
                    needs[i] = need
        return needs

    # ---- one step
    def forward(self, rt, meta, cache, logits_out=None):
        """float32 logits [wanted rows, vocab] (None when nothing is wanted); written into
        `logits_out` if that is given (it must have exactly that shape)."""
        with ops.stream_scope():
            return self._forward(rt, meta, cache, logits_out)

    def _forward(self, rt, meta, cache, logits_out=None):
        ctx = StepContext(rt=rt, meta=meta, cache=cache, logits_out=logits_out)
        x = self.embedding.forward(ctx, meta.token_ids)
        for i, e in enumerate(self.schedule):
            ctx.entry = i
            ctx.cache_entry = i if e.cache is None else e.cache
            ctx.owns_cache = e.cache is None
            # the norm that the residual stream meets after this block, for parts that can prepare it
            ctx.norm_after_block = None
            if i + 1 < len(self.schedule):
                first_norm = getattr(self.blocks[self.schedule[i + 1].layer], "first_norm", None)
                if first_norm is not None:
                    ctx.norm_after_block = (first_norm(), i + 1)
            # a block that knows nothing of norms handed from part to part must meet none
            ctx.handed = ctx.norm_ahead = None
            self.blocks[e.layer].forward(ctx, x)
        if meta.want_rows.shape[0] == 0:
            return None
        return self.head.forward(ctx, x, meta.want_rows)
