"""Random-weights mode: writes a model folder (config.json, model.safetensors) from a
configuration and a seed.

The reference gets random weights by constructing its model under torch.manual_seed
(tests/test_cache.py:34-35, bench/bench_paged.py:160-162); here the architecture's init plan
names every tensor, its shape and its rule, and the tensors are drawn in that order from one
seeded CPU generator, so the same (config, seed) always gives the same file.
"""

from __future__ import annotations

import os
from typing import Dict

import torch
from safetensors.torch import save_file

from ..config.model_config import write_config_json
from ..config.registry import architecture_of_config
from .loader import WEIGHTS_FILE


def random_tensors(config, seed: int, dtype: torch.dtype = torch.bfloat16, std_scale: float = 1.0
                   ) -> Dict[str, torch.Tensor]:
    """std_scale multiplies every standard deviation of the plan (gains stay centred on one)."""
    arch = architecture_of_config(config)
    gen = torch.Generator(device="cpu")
    gen.manual_seed(int(seed))
    tensors: Dict[str, torch.Tensor] = {}
    for name, shape, rule, scale in arch.init_plan(config):
        t = torch.empty(shape, dtype=torch.float32).normal_(0.0, scale * std_scale, generator=gen)
        if rule == "gain":
            t += 1.0
        elif rule != "normal":
            raise ValueError(f"unknown init rule {rule!r} for {name}")
        tensors[name] = t.to(dtype).contiguous()
    return tensors


def write_random_model(model_dir: str, config, seed: int, dtype: str = "bfloat16", std_scale: float = 1.0) -> str:
    os.makedirs(model_dir, exist_ok=True)
    write_config_json(model_dir, config)
    torch_dtype = {"bfloat16": torch.bfloat16, "float32": torch.float32}[dtype]
    save_file(random_tensors(config, seed, torch_dtype, std_scale), os.path.join(model_dir, WEIGHTS_FILE))
    return model_dir
