"""One registry from an architecture's name to its configuration class and model builder.

The reference has no registry: it whitelists `model_type` and serves both of
its families with one class (flow_engine/config.py:26, flow_engine/model.py:105).
Here config.json's `architectures[0]` (or, if absent, its `model_type`) selects
an entry; the entry's builder assembles a model out of parts.

What a configuration class must offer (the engine, the loader and the command
line read nothing else off it):

    from_dict(dict) -> config      parse config.json's own keys; raise ConfigError for what is not supported
    to_dict() -> dict              the keys back, so that a model folder can be written from a configuration
    describe() -> dict             what `inspect` and the log show
    architecture: str              the name it is registered under
    vocab_size: int                token ids are checked against it
    max_position_embeddings: int   the engine's `max_context` may not exceed it
    eos_token_ids: tuple[int]      tokens that end a request (merged from generation_config.json if present)
"""
from __future__ import annotations

from dataclasses import dataclass
import json
from pathlib import Path
from typing import Callable

from .model_config import ConfigError, with_generation_eos


@dataclass(frozen=True)
class Architecture:
    name: str                 # config.json "architectures"[0], e.g. "Qwen2ForCausalLM"
    model_type: str           # config.json "model_type", used when "architectures" is absent
    config_class: type        # has from_dict(dict) and to_dict()
    builder: Callable         # builder(config) -> parts.model.DecoderModel (weights unbound)


_ARCHITECTURES: dict[str, Architecture] = {}


def register_architecture(name, model_type, config_class, builder, replace=False):
    if name in _ARCHITECTURES and not replace:
        raise ValueError(f"architecture {name!r} is already registered")
    _ARCHITECTURES[name] = Architecture(name, model_type, config_class, builder)
    return _ARCHITECTURES[name]


def unregister_architecture(name):
    _ARCHITECTURES.pop(name, None)


def registered_architectures():
    _load_builtin()
    return sorted(_ARCHITECTURES)


def _load_builtin():
    # The built-in architecture registers itself on import.
    from .. import models  # noqa: F401


def architecture_for(config_dict) -> Architecture:
    _load_builtin()
    names = config_dict.get("architectures") or []
    if isinstance(names, str):
        names = [names]
    for name in names:
        if name in _ARCHITECTURES:
            return _ARCHITECTURES[name]
    if not names:
        for arch in _ARCHITECTURES.values():
            if arch.model_type == config_dict.get("model_type"):
                return arch
    raise ConfigError(
        f"no registered architecture for architectures={names!r} "
        f"model_type={config_dict.get('model_type')!r}; known: {sorted(_ARCHITECTURES)}")


def config_from_dict(config_dict):
    arch = architecture_for(config_dict)
    return arch.config_class.from_dict(config_dict)


def read_model_config(folder):
    """Parse FOLDER/config.json into its architecture's typed configuration."""
    folder = Path(folder)
    path = folder / "config.json"
    if not path.exists():
        raise ConfigError(f"{path} does not exist")
    config = config_from_dict(json.loads(path.read_text()))
    return with_generation_eos(config, folder)


def build_model(config, **options):
    """The architecture's model for CONFIG, assembled from parts, weights not yet bound.

    OPTIONS go to the architecture's builder (e.g. packed=False keeps q/k/v apart).
    """
    _load_builtin()
    arch = _ARCHITECTURES.get(getattr(config, "architecture", None))
    if arch is None:
        raise ConfigError(f"no registered architecture named {getattr(config, 'architecture', None)!r}")
    return arch.builder(config, **options)
