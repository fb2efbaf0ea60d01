"""Errors of the configuration layer."""


class ConfigError(ValueError):
    """config.json is missing a key, holds a bad value, or names an unsupported option."""


class UnsupportedArchitecture(ConfigError):
    """No registered architecture matches config.json."""
