"""The error every configuration parser and the architecture registry raise."""


class ConfigError(ValueError):
    """A configuration key is missing, has the wrong type or an unsupported value."""
