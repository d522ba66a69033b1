"""What every typed configuration shares: errors that name the field, and JSON reading."""

import json
import math
import os

INDEX_MAX = 2 ** 31 - 1          # sizes must fit the 32-bit indices of the kernels
MAX_LAYERS = 2 ** 18
MAX_CONFIG_BYTES = 16 * 2 ** 20


class ConfigError(ValueError):
    """A configuration value is missing, malformed or unsupported; displays ``family.field: reason``
    (the reference's ConfigError, src/models/config.rs:52-81)."""

    def __init__(self, family, field, reason):
        super().__init__(f"{family}.{field}: {reason}")
        self.family, self.field, self.reason = family, field, reason


class UnsupportedArchitecture(ValueError):
    """config.json names an architecture that no registered family runs."""


def read_config_json(model_dir):
    """The parsed ``config.json`` of a model folder (a regular file of bounded size)."""
    path = os.path.join(model_dir, "config.json")
    if not os.path.isfile(path):
        raise FileNotFoundError(f"{model_dir}: no config.json")
    if os.path.getsize(path) > MAX_CONFIG_BYTES:
        raise ValueError(f"{path}: larger than {MAX_CONFIG_BYTES} bytes")
    with open(path) as handle:
        data = json.load(handle)
    if not isinstance(data, dict):
        raise ValueError(f"{path}: the top level must be an object")
    return data


def unwrap_text_config(data):
    """Multimodal wrappers keep the language model's keys one level down
    (src/models/config.rs:214-229)."""
    for key in ("text_config", "language_config", "llm_config"):
        inner = data.get(key)
        if isinstance(inner, dict):
            merged = dict(inner)
            for outer in ("architectures", "model_type"):
                if outer not in merged and outer in data:
                    merged[outer] = data[outer]
            return merged
    return data


def take(data, family, field, kind, default, aliases=()):
    """data[field] (or an alias) checked to be of ``kind``; ``default`` when absent or null."""
    for key in (field,) + tuple(aliases):
        if key in data and data[key] is not None:
            value = data[key]
            break
    else:
        return default
    if kind is int:
        if isinstance(value, bool) or not isinstance(value, int):
            if isinstance(value, float) and value == int(value):
                return int(value)
            raise ConfigError(family, field, f"must be an integer, got {value!r}")
        return value
    if kind is float:
        if isinstance(value, bool) or not isinstance(value, (int, float)):
            raise ConfigError(family, field, f"must be a number, got {value!r}")
        return float(value)
    if kind is bool:
        if not isinstance(value, bool):
            raise ConfigError(family, field, f"must be true or false, got {value!r}")
        return value
    if kind is str:
        if not isinstance(value, str):
            raise ConfigError(family, field, f"must be a string, got {value!r}")
        return value
    raise TypeError(kind)


def positive_extent(family, field, value):
    if not (0 < value <= INDEX_MAX):
        raise ConfigError(family, field, "must be positive and fit the portable integer index range")


def positive_finite(family, field, value):
    if not (math.isfinite(value) and value > 0):
        raise ConfigError(family, field, "must be finite and greater than zero")
