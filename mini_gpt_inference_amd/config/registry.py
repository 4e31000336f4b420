"""One registry from an architecture's name to how its model is built."""

from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Callable, Dict, List, Mapping, Tuple


@dataclass(frozen=True)
class Architecture:
    name: str
    config_from_json: Callable[[Mapping[str, Any]], Any]   # config.json dict -> typed config
    model_spec: Callable[[Any], Any]                        # typed config -> parts.model.ModelSpec
    init_plan: Callable[[Any], List[Tuple[str, Tuple[int, ...], str, float]]]
    # init_plan: (tensor name, shape, rule, scale) in the order tensors are drawn in random-weights mode


_ARCHITECTURES: Dict[str, Architecture] = {}


def register_architecture(arch: Architecture) -> None:
    if arch.name in _ARCHITECTURES and _ARCHITECTURES[arch.name] is not arch:
        raise ValueError(f"architecture {arch.name!r} is already registered")
    _ARCHITECTURES[arch.name] = arch


def get_architecture(name: str) -> Architecture:
    _load_builtin()
    if name not in _ARCHITECTURES:
        raise KeyError(f"unknown architecture {name!r}; registered: {sorted(_ARCHITECTURES)}")
    return _ARCHITECTURES[name]


def architecture_names() -> List[str]:
    _load_builtin()
    return sorted(_ARCHITECTURES)


def architecture_of(raw_config: Mapping[str, Any]) -> Architecture:
    """The architecture a config.json names under `architecture` (or `model_type`)."""
    name = raw_config.get("architecture", raw_config.get("model_type"))
    if not isinstance(name, str):
        raise KeyError("config.json names no architecture (key 'architecture')")
    return get_architecture(name)


def _load_builtin() -> None:
    from ..models import gpt2_mini  # noqa: F401  (registers itself)
