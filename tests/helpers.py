"""Tiny configurations, model folders and tolerances shared by the tests."""

from __future__ import annotations

import os
from typing import Callable, Dict, Optional

import numpy as np
import torch
from safetensors.torch import save_file

from mini_gpt_inference_amd import GPTConfig
from mini_gpt_inference_amd.config.model_config import write_config_json
from mini_gpt_inference_amd.weights.random_init import random_tensors

# Two tiny configurations that differ in every size and option (layers, width, heads, head size,
# vocabulary, positions, bias, eps), plus a long-context one for far-key tests.
CONFIGS: Dict[str, GPTConfig] = {
    "A": GPTConfig("gpt2-mini", n_layer=2, n_embd=64, n_head=4, vocab_size=257, block_size=64, bias=True,
                   layer_norm_eps=1e-5),
    "B": GPTConfig("gpt2-mini", n_layer=3, n_embd=96, n_head=3, vocab_size=503, block_size=128, bias=False,
                   layer_norm_eps=1e-6),
    "LONG": GPTConfig("gpt2-mini", n_layer=1, n_embd=48, n_head=1, vocab_size=61, block_size=640, bias=True,
                      layer_norm_eps=1e-3),
}
SEEDS = {"A": 0, "B": 1, "LONG": 2}
# The init rule's standard deviations give nearly uniform attention and tiny logits, which hides
# faults; the tests scale them up so that softmax is peaked and every path carries signal.
STD_SCALE = {"A": 5.0, "B": 5.0, "LONG": 6.0}

# Tolerances, fixed before any kernel was measured.  float32: summation order only.  bfloat16:
# activations and weights carry 8 bits of mantissa (relative 2^-9 per rounding, a handful of
# roundings per layer), the reference's own half-precision bound is 2e-2 (tests/test_triton.py:101).
TOL = {"float32": 2e-5, "bfloat16": 2e-2}


def write_model(path: str, name: str, edit: Optional[Callable[[Dict[str, torch.Tensor]], None]] = None,
                dtype: torch.dtype = torch.bfloat16) -> str:
    cfg = CONFIGS[name]
    tensors = random_tensors(cfg, SEEDS[name], dtype, STD_SCALE[name])
    if edit is not None:
        edit(tensors)
    os.makedirs(path, exist_ok=True)
    write_config_json(path, cfg)
    save_file({k: v.contiguous() for k, v in tensors.items()}, os.path.join(path, "model.safetensors"))
    return path


def assert_close(got, want, dtype: str, what: str = "") -> None:
    """max |got - want| <= TOL[dtype] * max(1, max |want|)."""
    got = torch.as_tensor(np.asarray(got.detach().cpu() if isinstance(got, torch.Tensor) else got)).double()
    want = torch.as_tensor(np.asarray(want.detach().cpu() if isinstance(want, torch.Tensor) else want)).double()
    assert got.shape == want.shape, f"{what}: shape {tuple(got.shape)} vs {tuple(want.shape)}"
    assert torch.isfinite(got).all(), f"{what}: non-finite values in the engine's result"
    scale = max(1.0, float(want.abs().max()))
    err = float((got - want).abs().max())
    assert err <= TOL[dtype] * scale, f"{what}: max error {err:.3e} > {TOL[dtype]:.0e} * {scale:.3g}"


def random_ids(rng: np.random.Generator, vocab: int, n: int):
    return rng.integers(0, vocab, n).tolist()
