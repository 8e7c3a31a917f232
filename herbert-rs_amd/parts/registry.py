"""Registries of parts: kind -> class, one per category.

A part class is registered with `@register(category, kind)` and built with
`build(category, spec, **context)`. The categories are "mixer",
"feed_forward", "norm", "position", "block", "embedding" and "head"; a test
or a user may add kinds without touching this package.
"""
from ..errors import ConfigError

CATEGORIES = ("mixer", "feed_forward", "norm", "position", "block", "embedding", "head")
_REGISTRY = {c: {} for c in CATEGORIES}


def register(category, kind):
    if category not in _REGISTRY:
        raise ConfigError(f"unknown part category {category!r}")

    def deco(cls):
        _REGISTRY[category][kind] = cls
        cls.kind = kind
        return cls
    return deco


def registered(category):
    return sorted(_REGISTRY[category])


def build(category, spec, **context):
    """An instance of the part that `spec` names, with its parameters and the given context."""
    try:
        cls = _REGISTRY[category][spec.kind]
    except KeyError:
        raise ConfigError(f"unknown {category} {spec.kind!r}; registered: "
                          f"{', '.join(registered(category))}") from None
    return cls(**spec.params, **context)
