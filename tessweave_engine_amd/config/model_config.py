"""What every architecture's typed configuration shares: the error a config.json is refused with and
the EOS ids (flow_engine/config.py:54-62: generation_config.json overrides config.json's).

An architecture's own configuration class lives beside its model builder (`models/`); what the rest of
the package reads off such a class is listed in `registry.py`.
"""
from __future__ import annotations

from dataclasses import replace
import json
from pathlib import Path


class ConfigError(ValueError):
    """config.json asks for something this engine does not implement."""


def eos_tuple(value):
    if value is None:
        return ()
    if isinstance(value, bool):
        raise ConfigError("eos_token_id must be an int, a list of ints or null")
    if isinstance(value, int):
        return (value,)
    return tuple(int(v) for v in value)


def with_generation_eos(config, folder):
    """generation_config.json's eos_token_id replaces config.json's when present."""
    generation = Path(folder) / "generation_config.json"
    if generation.exists():
        eos = json.loads(generation.read_text()).get("eos_token_id")
        if eos is not None:
            config = replace(config, eos_token_ids=eos_tuple(eos))
    return config
