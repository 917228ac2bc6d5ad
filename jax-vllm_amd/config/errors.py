class ConfigError(ValueError):
    """A configuration file or value is missing, mistyped or inconsistent."""
