"""The error of every configuration: a config.json that cannot be read, parsed or honoured, or that names an
architecture the registry does not know.  It belongs to no architecture; their configuration classes raise it."""


class ConfigError(ValueError):
    pass
