"""Reading and writing config.json, for any architecture.

What the keys mean is the architecture's business: its module under models/ has the typed
configuration class and registers how to read it from, and write it to, this file
(config.registry.Architecture).  The reference has one configuration dataclass and no file
format for it (src/minigpt_infer/config.py:10-18; a checkpoint carries it, loader.py:63-85).
"""

from __future__ import annotations

import json
import os
from typing import Any


class ConfigError(ValueError):
    """A config.json that cannot describe a model of the named architecture."""


def read_config_json(model_dir: str) -> dict[str, Any]:
    path = os.path.join(model_dir, "config.json")
    if not os.path.isfile(path):
        raise ConfigError(f"no config.json in {model_dir}")
    with open(path, "r", encoding="utf-8") as fh:
        raw = json.load(fh)
    if not isinstance(raw, dict):
        raise ConfigError(f"{path} does not hold a JSON object")
    return raw


def write_config_json(model_dir: str, config: Any) -> None:
    """Writes the typed configuration of any registered architecture (config.architecture names it)."""
    from .registry import architecture_of_config

    raw = dict(architecture_of_config(config).config_to_json(config))
    os.makedirs(model_dir, exist_ok=True)
    with open(os.path.join(model_dir, "config.json"), "w", encoding="utf-8") as fh:
        json.dump(raw, fh, indent=2, sort_keys=True)
        fh.write("\n")
