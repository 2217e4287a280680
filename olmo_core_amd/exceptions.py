"""Error types raised at the configuration boundary (reference: src/olmo_core/exceptions.py:1-27)."""


class OLMoError(Exception):
    """Base class for errors raised by this package."""


class OLMoConfigurationError(OLMoError):
    """An invalid or inconsistent configuration."""


class MI8KernelError(RuntimeError):
    """A non-zero status came back from the native library."""
