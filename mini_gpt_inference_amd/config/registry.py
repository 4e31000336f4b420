"""One registry from an architecture's name to how its model is built.

An architecture is a module under models/ that calls register_architecture once.  Every module
found there is imported when a name is first looked up, so adding an architecture is adding a
file; nothing here names one.  What the framework asks of an architecture's typed configuration
is little: an attribute `architecture` that holds the registered name (config.json carries it
under the same key), and the two conversions below.
"""

from __future__ import annotations

import importlib
import pkgutil
from dataclasses import dataclass
from typing import Any, Callable, Dict, List, Mapping, Set, Tuple


@dataclass(frozen=True)
class Architecture:
    name: str
    config_from_json: Callable[[Mapping[str, Any]], Any]   # config.json dict -> typed config
    model_spec: Callable[[Any], Any]                        # typed config -> parts.model.ModelSpec
    init_plan: Callable[[Any], List[Tuple[str, Tuple[int, ...], str, float]]]
    # init_plan: (tensor name, shape, rule, scale) in the order tensors are drawn in random-weights mode
    config_to_json: Callable[[Any], Mapping[str, Any]] = lambda config: config.to_json_dict()
    # typed config -> the dict that config.json holds (flat; carries "architecture": name)


_ARCHITECTURES: Dict[str, Architecture] = {}
_SCANNED: Set[str] = set()      # modules under models/ imported so far


def register_architecture(arch: Architecture) -> None:
    if arch.name in _ARCHITECTURES and _ARCHITECTURES[arch.name] is not arch:
        raise ValueError(f"architecture {arch.name!r} is already registered")
    _ARCHITECTURES[arch.name] = arch


def get_architecture(name: str) -> Architecture:
    if name not in _ARCHITECTURES:
        _load_models()
    if name not in _ARCHITECTURES:
        raise KeyError(f"unknown architecture {name!r}; registered: {sorted(_ARCHITECTURES)}")
    return _ARCHITECTURES[name]


def architecture_names() -> List[str]:
    _load_models()
    return sorted(_ARCHITECTURES)


def architecture_of(raw_config: Mapping[str, Any]) -> Architecture:
    """The architecture a config.json names under `architecture` (or `model_type`)."""
    name = raw_config.get("architecture", raw_config.get("model_type"))
    if not isinstance(name, str):
        raise KeyError("config.json names no architecture (key 'architecture')")
    return get_architecture(name)


def architecture_of_config(config: Any) -> Architecture:
    """The architecture of a typed configuration: the one its `architecture` attribute names."""
    name = getattr(config, "architecture", None)
    if not isinstance(name, str):
        raise TypeError(f"{type(config).__name__} has no attribute 'architecture' that names its architecture")
    return get_architecture(name)


def _load_models() -> None:
    """Imports every module of the models package that has not been imported yet (each registers
    itself).  The package's search path is read anew at every call: a module that appears later, or
    a folder appended to models.__path__, is found at the next lookup of an unknown name."""
    from .. import models

    for info in pkgutil.iter_modules(models.__path__):
        if info.name.startswith("_") or info.name in _SCANNED:
            continue
        _SCANNED.add(info.name)
        importlib.import_module(f"{models.__name__}.{info.name}")
