"""Typed errors of the engine.

The names follow the reference where it has them (exceptions.py:1-19:
`OutOfMemoryError`, `EngineNotRunningError`, `RequestFailedError`).
"""


class OutOfMemoryError(RuntimeError):
    """The cache has too few free pages (or state slots) for what was asked."""


class EngineNotRunningError(RuntimeError):
    """A request was given to a scheduler whose engine has stopped."""


class RequestFailedError(RuntimeError):
    """The engine failed while a request was in flight."""


class ConfigError(ValueError):
    """A config.json is missing a key the architecture needs, or holds a bad value."""


class WeightLoadError(ValueError):
    """A checkpoint does not fit the model: missing, unexpected or wrongly shaped tensors."""


class KernelShapeError(ValueError):
    """A kernel was asked for a size it does not take; it refuses instead of guessing."""


class ExtensionMissingError(RuntimeError):
    """The HIP library is not built and cannot be built here; there is no fallback."""
