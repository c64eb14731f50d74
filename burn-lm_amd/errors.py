"""Errors that several parts of the library raise, kept apart from any one architecture."""


class ConfigError(ValueError):
    """config.json is missing, is no JSON, lacks a key, holds a value of the wrong kind, or asks for
    something the architecture does not have."""
