"""Reads a model folder (config.json + model.safetensors) into device tensors by tensor name.

Storage rule: matrices and tables are kept in the compute dtype, which is bfloat16 when
serving; gains and biases are kept in float32 (an exact widening of what a bfloat16 file
holds); a matrix or table that the file stores in 32-bit stays in 32-bit; integer tables
become int32.  On the 32-bit path everything is widened to float32.

The reference loads a training checkpoint with torch.load and load_state_dict(strict=False),
then raises on any missing or unexpected key (src/minigpt_infer/loader.py:102-118); here the
container is safetensors and the one error also lists wrong shapes.
"""

from __future__ import annotations

import os
from typing import Dict, List, Mapping, Tuple

import torch
from safetensors import safe_open

from ..config.model_config import read_config_json
from ..config.registry import Architecture, architecture_of
from ..parts.base import VECTOR, WeightRequest

WEIGHTS_FILE = "model.safetensors"
# DDP and torch.compile wrap state-dict keys (src/minigpt_infer/loader.py:107-110)
_PREFIXES = ("module.", "_orig_mod.")


class WeightError(RuntimeError):
    """The tensors of a model folder do not match what its config.json describes."""


def strip_prefix(names: Mapping[str, object], prefix: str) -> Dict[str, object]:
    """Strips `prefix` from the keys that carry it, if any key does
    (src/minigpt_infer/loader.py:35-38; mixed keys: tests/test_loader.py:29-36)."""
    if not any(k.startswith(prefix) for k in names):
        return dict(names)
    return {(k[len(prefix):] if k.startswith(prefix) else k): v for k, v in names.items()}


def _target_dtype(stored: torch.dtype, role: str, compute: torch.dtype) -> torch.dtype:
    if not stored.is_floating_point:
        return torch.int32
    if compute == torch.float32 or role == VECTOR:
        return torch.float32
    if stored in (torch.float32, torch.float64):
        return torch.float32          # a tensor stored in 32-bit stays so
    return torch.bfloat16


def load_tensors(model_dir: str, wanted: Mapping[str, WeightRequest], compute_dtype: torch.dtype,
                 device: torch.device, tied: Mapping[str, str] = ()) -> Dict[str, torch.Tensor]:
    """Loads exactly the tensors in `wanted`.  `tied` maps an optional duplicate name to the tensor
    it must equal (the reference's state dict lists the tied head twice, model.py:128-130)."""
    path = os.path.join(model_dir, WEIGHTS_FILE)
    if not os.path.isfile(path):
        raise WeightError(f"no {WEIGHTS_FILE} in {model_dir}")
    tied = dict(tied)
    out: Dict[str, torch.Tensor] = {}
    with safe_open(path, framework="pt", device="cpu") as fh:
        by_name: Dict[str, str] = {k: k for k in fh.keys()}   # stripped name -> name in the file
        for prefix in _PREFIXES:
            by_name = strip_prefix(by_name, prefix)
        missing = sorted(n for n in wanted if n not in by_name)
        unexpected = sorted(n for n in by_name if n not in wanted and n not in tied)
        wrong: List[Tuple[str, Tuple[int, ...], Tuple[int, ...]]] = []
        for name, req in wanted.items():
            if name in by_name:
                shape = tuple(fh.get_slice(by_name[name]).get_shape())
                if shape != tuple(req.shape):
                    wrong.append((name, tuple(req.shape), shape))
        if missing or unexpected or wrong:
            lines = [f"{path} does not match the model that config.json describes:"]
            if missing:
                lines.append(f"  missing tensors ({len(missing)}): {missing}")
            if unexpected:
                lines.append(f"  unexpected tensors ({len(unexpected)}): {unexpected}")
            for name, want, got in wrong:
                lines.append(f"  wrong shape: {name} should be {list(want)}, file has {list(got)}")
            raise WeightError("\n".join(lines))
        for name, req in wanted.items():
            t = fh.get_tensor(by_name[name])
            out[name] = t.to(_target_dtype(t.dtype, req.role, compute_dtype)).contiguous().to(device)
        for dup, base in tied.items():
            if dup in by_name:
                t = fh.get_tensor(by_name[dup])
                ref = fh.get_tensor(by_name[base])
                if t.shape != ref.shape or not torch.equal(t, ref):
                    raise WeightError(f"{dup} is stored beside {base} but differs from it; they are one tensor")
    return out


def load_model(model_dir: str, dtype: str, device: str = "cuda"):
    """config.json -> architecture -> model with its tensors on the device.
    Returns (model, config, architecture)."""
    from ..parts.model import DecoderModel

    raw = read_config_json(model_dir)
    arch: Architecture = architecture_of(raw)
    config = arch.config_from_json(raw)
    model = DecoderModel(arch.model_spec(config))
    compute = {"bfloat16": torch.bfloat16, "float32": torch.float32}[dtype]
    tensors = load_tensors(model_dir, model.weight_requests(), compute, torch.device(device),
                           tied=dict(model.spec.tied_aliases))
    model.bind(tensors)
    return model, config, arch
