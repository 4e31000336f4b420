"""Typed model configuration, read from the architecture's own config.json keys.

The keys are the fields of the reference's ``GPTConfig`` dataclass
(src/minigpt_infer/config.py:10-18): vocab_size, block_size, n_layer, n_head,
n_embd, dropout, bias.  ``layer_norm_eps`` is added here because the reference
leaves it at ``nn.LayerNorm``'s default (src/minigpt_infer/model.py:107,109,127)
and a model folder has to be able to say otherwise.
"""

from __future__ import annotations

import json
import os
from dataclasses import asdict, dataclass, fields
from typing import Any, Mapping

# Keys a config.json may carry that the engine reads past: the reference forces
# dropout to 0 at inference (src/minigpt_infer/loader.py:58).
_IGNORED_KEYS = {"dropout", "model_type", "torch_dtype"}


class ConfigError(ValueError):
    """A config.json that cannot describe a model of the named architecture."""


@dataclass(frozen=True)
class GPTConfig:
    """GPT-2-style dense decoder (src/minigpt_infer/model.py:118-130)."""

    architecture: str
    n_layer: int
    n_embd: int
    n_head: int
    vocab_size: int
    block_size: int          # rows of the learned position table = most positions
    bias: bool               # biases on every Linear and every LayerNorm
    layer_norm_eps: float = 1e-5

    def __post_init__(self) -> None:
        for name in ("n_layer", "n_embd", "n_head", "vocab_size", "block_size"):
            value = getattr(self, name)
            if not isinstance(value, int) or isinstance(value, bool) or value <= 0:
                raise ConfigError(f"{name} must be a positive integer, got {value!r}")
        if not isinstance(self.bias, bool):
            raise ConfigError(f"bias must be true or false, got {self.bias!r}")
        if not (isinstance(self.layer_norm_eps, float) and self.layer_norm_eps > 0.0):
            raise ConfigError(f"layer_norm_eps must be a positive float, got {self.layer_norm_eps!r}")
        # src/minigpt_infer/model.py:39
        if self.n_embd % self.n_head != 0:
            raise ConfigError(
                f"n_embd ({self.n_embd}) is not divisible by n_head ({self.n_head})"
            )

    @property
    def head_dim(self) -> int:
        return self.n_embd // self.n_head

    def to_json_dict(self) -> dict[str, Any]:
        return asdict(self)

    @classmethod
    def from_json_dict(cls, raw: Mapping[str, Any]) -> "GPTConfig":
        known = {f.name for f in fields(cls)}
        data = dict(raw)
        if "architecture" not in data and "model_type" in data:
            data["architecture"] = data["model_type"]
        unknown = sorted(k for k in data if k not in known and k not in _IGNORED_KEYS
                         and not k.startswith("_"))
        if unknown:
            raise ConfigError(f"config.json has keys this architecture does not know: {unknown}")
        required = [f.name for f in fields(cls) if f.name != "layer_norm_eps"]
        missing = [k for k in required if k not in data]
        if missing:
            raise ConfigError(f"config.json lacks required keys: {missing}")
        kwargs = {k: data[k] for k in known if k in data}
        if "layer_norm_eps" in kwargs:
            kwargs["layer_norm_eps"] = float(kwargs["layer_norm_eps"])
        return cls(**kwargs)


def read_config_json(model_dir: str) -> dict[str, Any]:
    path = os.path.join(model_dir, "config.json")
    if not os.path.isfile(path):
        raise ConfigError(f"no config.json in {model_dir}")
    with open(path, "r", encoding="utf-8") as fh:
        raw = json.load(fh)
    if not isinstance(raw, dict):
        raise ConfigError(f"{path} does not hold a JSON object")
    return raw


def write_config_json(model_dir: str, config: GPTConfig) -> None:
    os.makedirs(model_dir, exist_ok=True)
    with open(os.path.join(model_dir, "config.json"), "w", encoding="utf-8") as fh:
        json.dump(config.to_json_dict(), fh, indent=2, sort_keys=True)
        fh.write("\n")
