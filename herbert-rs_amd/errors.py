"""Error kinds of the library.

They mirror the reference's error enum (crates/core/src/error.rs:8-36): one
class for each of its kinds that this library can raise, all under
`HerbertError`.
"""


class HerbertError(Exception):
    """Root of every error this library raises on purpose."""


class ConfigError(HerbertError):
    """config.json is missing a key, holds a bad value or names an unknown architecture."""


class ModelLoadError(HerbertError):
    """The weights do not fit the configuration (missing, unexpected, wrong shape or dtype)."""


class BackendError(HerbertError):
    """The GPU side failed or cannot run the request (extension missing, size refused)."""


class CacheError(HerbertError):
    """Slots or pages are exhausted, or a slot is used in a way its state forbids."""


class RequestError(HerbertError):
    """A step or a generation request is malformed (empty sequence, bad token id, too long)."""


class NeedsEagerStep(BackendError):
    """While a step is recorded into a graph, something needs memory that it does not have yet
    (a scratch buffer, room for a list): nothing can be allocated inside a recording, so the step
    has to run outside one first. The engine catches this and does that; nobody else sees it."""
