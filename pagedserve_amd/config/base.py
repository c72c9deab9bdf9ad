"""What every architecture's configuration shares: the error type, reading ``config.json``,
and checked access to its keys.  Nothing here knows an architecture."""

import json
import os


class ConfigError(ValueError):
    """A config.json that this engine cannot run, with the reason."""


def read_config_json(folder) -> dict:
    path = os.path.join(folder, "config.json")
    if not os.path.isfile(path):
        raise ConfigError(f"{folder!r} holds no config.json")
    with open(path) as handle:
        raw = json.load(handle)
    if not isinstance(raw, dict):
        raise ConfigError(f"{path} does not hold a JSON object")
    return raw


def require_int(raw, key, default=None, minimum=1):
    """``raw[key]`` (or ``default``) as an integer of at least ``minimum``."""
    value = raw.get(key, default)
    if value is None:
        raise ConfigError(f"config.json lacks '{key}'")
    if isinstance(value, bool) or not isinstance(value, int):
        raise ConfigError(f"config.json '{key}' must be an integer, got {value!r}")
    if value < minimum:
        raise ConfigError(f"config.json '{key}' must be >= {minimum}, got {value}")
    return value
