"""The error every configuration class raises for a config.json it cannot run."""


class ConfigError(ValueError):
    """config.json cannot be run by this engine; the message names the key."""
