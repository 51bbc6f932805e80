class ConfigError(ValueError):
    """A config.json that the architecture cannot be built from."""
