"""How an architecture's checkpoints spell their tensor names.

The generic reader knows no spelling of its own: an architecture registers a
NameMap beside its configuration class, and the reader asks it for the name a
stored tensor has in the model's own terms and for the tensors a fused one is
cut into. The reference does both inside its one loader
(crates/backends/backend_common/src/loader_common.rs:423-451 prefixes and
aliases, :1469-1528 fused tensors); which spellings exist is a fact about a
family of checkpoints, so here it is data of the architecture.
"""
from dataclasses import dataclass, field
from typing import Dict, Tuple


@dataclass(frozen=True)
class NameMap:
    """prefixes: (stored prefix, model's prefix) pairs, the first that matches is applied.
    bare_prefix / bare_starts: a stored name that begins with one of `bare_starts` and has no
    known prefix gets `bare_prefix` in front.
    suffixes: (stored suffix, model's suffix) pairs.
    layer_prefix: what precedes a layer's number in the model's names ("model.layers.").
    layer_aliases: within a layer, stored spelling -> the model's.
    fused: within a layer, a fused tensor's name -> the names its rows are cut into, in order.
    """
    prefixes: Tuple[Tuple[str, str], ...] = ()
    bare_prefix: str = ""
    bare_starts: Tuple[str, ...] = ()
    keep_starts: Tuple[str, ...] = ()
    suffixes: Tuple[Tuple[str, str], ...] = ()
    layer_prefix: str = ""
    layer_aliases: Dict[str, str] = field(default_factory=dict)
    fused: Dict[str, Tuple[str, ...]] = field(default_factory=dict)

    def __hash__(self):
        return id(self)

    def canonical(self, name):
        """A stored tensor's name as the model asks for it."""
        for stored, own in self.prefixes:
            if name.startswith(stored):
                name = own + name[len(stored):]
                break
        else:
            if self.bare_starts and not name.startswith(self.keep_starts) \
                    and name.startswith(self.bare_starts):
                name = self.bare_prefix + name
        for stored, own in self.suffixes:
            if name.endswith(stored):
                name = name[:-len(stored)] + own
        if self.layer_prefix and name.startswith(self.layer_prefix):
            number, _, rest = name[len(self.layer_prefix):].partition(".")
            if rest in self.layer_aliases:
                name = f"{self.layer_prefix}{number}.{self.layer_aliases[rest]}"
        return name

    def fused_targets(self, name, needs):
        """For a fused tensor's (canonical) name: the names its rows are cut into, if the model
        asks for all of them; else None."""
        for suffix, parts in self.fused.items():
            if name.endswith("." + suffix):
                prefix = name[:-len(suffix)]
                targets = [prefix + p for p in parts]
                if all(t in needs for t in targets):
                    return targets
        return None


AS_STORED = NameMap()
