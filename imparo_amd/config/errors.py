"""Errors a configuration can raise.

Four classes, the same four the reference plans fail with
(/root/reference/crates/imparo-model/src/lib.rs:582-598: UnknownArchitecture,
MissingMetadata, BadMetadata, Inconsistent).
"""


class ConfigError(ValueError):
    """Base of every configuration failure."""


class UnknownArchitecture(ConfigError):
    """config.json names an architecture no builder is registered for."""


class MissingKey(ConfigError):
    """A required config.json key is absent."""


class BadValue(ConfigError):
    """A key is present but its value has the wrong type or range."""


class Inconsistent(ConfigError):
    """Keys are individually valid but contradict each other."""
